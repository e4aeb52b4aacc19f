#!/usr/bin/env python3
"""Benchmark of the fused MoE forward on one MI355X.

A step is one moe_forward call (gate -> slots -> expert FFN -> combine) on one batch of synthetic tokens already
resident in HBM.  Headline workload: the Mixtral-shape configuration (S=8192, H=4096, I=14336, E=8, top-2, SwiGLU,
bf16, dropless).  Prints one JSON line:
  value         tokens/s of the whole layer, from the wall clock around the K timed steps
  roofline      the expert-FFN kernel (the dominant launch) against the bf16 MFMA peak -- or the HBM peak for the fp8
                decode shape -- from hipEvents recorded around that kernel inside the same K steps
  cpu_baseline  the layer written with libtorch CPU ops (the role the reference reserves in torching.cuh:7-11 and
                leaves empty), timed on this box's host cores on a bounded token sample; the CPU oracle's timing on
                the same sample is given beside it
  workloads     the other configurations (decode fp8, mid, fine-grained), each with its own step time, stage times
                and roofline, measured the same way in the same run
"""
import argparse
import hashlib
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_F32_TFLOPS = 157.3
PEAK_FP8_TFLOPS = 5000.0      # MI355X dense fp8 MFMA: what bounds a layer whose both GEMM operands are e4m3 (option fp8_mfma)
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E

# Bytes per FFN-kernel launch that crossed the L2 <-> memory-fabric boundary, from two rocprofv3 --pmc runs of this
# script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter showed for a 1 GiB
# device copy in the same run (--calibrate-copy).  Each entry names the summary under profiles/ it comes from and the
# digest of the kernel sources it was collected with: when the sources have changed since, the figure is withheld.
BF16_SOURCES = ("ffn_bf16.hip", "ffn_bf16_slab_steady.inc", "ffn_common.hpp", "route.hip")
FP8_SOURCES = ("ffn_fp8.hip", "ffn_common.hpp", "route.hip")
FP8_TILE_SOURCES = ("ffn_fp8_tile.hip", "ffn_common.hpp", "route.hip")
WIDEN_SOURCES = BF16_SOURCES + ("quant.hip",)
F32_TILE_SOURCES = ("ffn_f32_tile.hip", "ffn_common.hpp", "route.hip")
FP8_MFMA_SOURCES = FP8_TILE_SOURCES + ("quant.hip",)
MEASURED_TRAFFIC = {
    "mixtral": {"bytes": 18.13e9, "sources": BF16_SOURCES, "kernel_digest": "3c477f620de7",
                "profile": "profiles/ffn_persistent_kernel_bf16_mixtral_c3_hbm_traffic.txt"},
    "mid": {"bytes": 0.8081e9, "sources": BF16_SOURCES, "kernel_digest": "3c477f620de7",
            "profile": "profiles/ffn_persistent_kernel_bf16_mid_c2_hbm_traffic.txt"},
    "finegrained": {"bytes": 3.336e9, "sources": BF16_SOURCES, "kernel_digest": "3c477f620de7",
                    "profile": "profiles/ffn_persistent_kernel_bf16_finegrained_c4_hbm_traffic.txt"},
    "decode_fp8": {"bytes": 9.909e9, "sources": FP8_SOURCES, "kernel_digest": "47ddccc0e23f",
                   "profile": "profiles/ffn_persistent_fp8_kernel_decode_c5_hbm_traffic.txt"},
    # a single-expert fp32 layer runs as two launches (one per projection); the figure is their sum
    "reference_default": {"bytes": 0.9158e9, "sources": F32_TILE_SOURCES, "kernel_digest": "3e84a4ffa895", "ffn_mode": 1,
                          "profile": "profiles/ffn_tiled_f32_tile_kernel_reference_default_hbm_traffic.txt"},
    # the widening pass and the bf16 queue kernel together (what the layer's FFN stage launches by default) ...
    "prefill_fp8": {"bytes": 23.05e9, "sources": WIDEN_SOURCES, "kernel_digest": "967a29900dec",
                    "profile": "profiles/widen_plus_ffn_persistent_kernel_prefill_fp8_hbm_traffic.txt"},
    # ... the e4m3 tile GEMM on the same layer (option fp8_widen = 0) ...
    "prefill_fp8/e4m3_tile": {"bytes": 26.29e9, "sources": FP8_TILE_SOURCES, "kernel_digest": "5197e02dde8f",
                              "profile": "profiles/ffn_persistent_fp8_tile_kernel_prefill_fp8_hbm_traffic.txt"},
    # ... and the e4m3 x e4m3 plan (option fp8_mfma = 1): two quantising passes and two GEMM launches
    "prefill_fp8/e4m3_mfma": {"bytes": 14.60e9, "sources": FP8_MFMA_SOURCES, "kernel_digest": "7f390a4e2f33", "ffn_mode": 1,
                              "profile": "profiles/ffn_tiled_fp8_mfma_kernel_prefill_fp8_hbm_traffic.txt"},
}


def kernel_digest(sources=BF16_SOURCES):
    h = hashlib.sha256()
    for name in sources:
        with open(os.path.join(ROOT, "cuplayground_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:12]


def stats(samples):
    if not samples:
        return None
    return {"mean": round(statistics.fmean(samples), 5), "median": round(statistics.median(samples), 5),
            "min": round(min(samples), 5), "n": len(samples)}


def measure(name, steps, warmup, seed, ffn_mode, calibrate_copy=False, balanced_routing=False, options=None,
            other_plans=False):
    """Runs one workload; returns (result dict, layer, device operands, output tensor, routing tensors)."""
    import torch
    import cuplayground_amd as moe
    from cuplayground_amd import api, workloads as wl

    w = wl.WORKLOADS[name]
    c = w.config
    layer = moe.MoELayer(c, ffn_mode=ffn_mode, options=options)
    dev = wl.make_device_inputs(w, seed)
    if balanced_routing:
        wl.balance_routing(c, dev)
    out = torch.empty(c.tokens, c.hidden_size, dtype=layer.act_dtype, device="cuda")
    if calibrate_copy:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)              # reads 1 GiB and writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(warmup):
        layer.forward(dev["x"], dev, out=out)
    torch.cuda.synchronize()
    # the timed region behind `value`: exactly `steps` calls, nothing else on the stream
    t0 = time.perf_counter()
    for _ in range(steps):
        layer.forward(dev["x"], dev, out=out)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps
    # the same `steps` calls again with hipEvents around every stage (recorded by the library on this stream) and
    # around every call: kernel durations, stage breakdown, medians.  The event records themselves cost about 15 us
    # per call, which is why they stay out of the region above.
    layer.set_stage_timing(True)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t2 = time.perf_counter()
    for a, b in ev:
        a.record()
        layer.forward(dev["x"], dev, out=out)
        b.record()
    torch.cuda.synchronize()
    t3 = time.perf_counter()
    stage_mean = layer.stage_ms()
    samples = layer.stage_samples()
    layer.set_stage_timing(False)
    step_ms = [a.elapsed_time(b) for a, b in ev]
    ms_per_step_events = (t3 - t2) * 1e3 / steps

    # the same `steps` calls once more as replays of a HIP graph holding one forward call: what a serving loop that
    # captures the layer pays per step (launch-bound shapes gain; the others show that capture costs nothing)
    graph_ms = graph_err = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            layer.forward(dev["x"], dev, out=out)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            layer.forward(dev["x"], dev, out=out)
        for _ in range(warmup):
            graph.replay()
        torch.cuda.synchronize()
        t4 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t4) * 1e3 / steps
        del graph
    except Exception as e:        # reported, never fatal: the figures above do not depend on it
        graph_err = "%s: %s" % (type(e).__name__, e)

    # a plan that derives operands from the weights in every call (the bf16 copies of an e4m3 layer on the widening
    # plan): the same steps once more with those operands made once by moe_prepare_weights and handed in
    prepared_ms = None
    if layer.prepared_bytes:
        ready = dict(dev, prepared=layer.prepare_weights(dev))
        for _ in range(warmup):
            layer.forward(dev["x"], ready, out=out)
        torch.cuda.synchronize()
        t5 = time.perf_counter()
        for _ in range(steps):
            layer.forward(dev["x"], ready, out=out)
        torch.cuda.synchronize()
        prepared_ms = (time.perf_counter() - t5) * 1e3 / steps
        del ready

    # the same steps with e4m3 activations on the fp8 matrix instruction (option fp8_mfma: other arithmetic, opt-in;
    # reported beside the default plan of a prefill-sized e4m3 layer, never in its place)
    fp8_mfma_ms = None
    if other_plans and c.torch_dtype == api.DTYPE_FP8 and w.bound == "mfma" and (options or {}).get("fp8_mfma") is None:
        alt = moe.MoELayer(c, ffn_mode=ffn_mode, options=dict(options or {}, fp8_mfma=1))
        for _ in range(warmup):
            alt.forward(dev["x"], dev, out=out)
        torch.cuda.synchronize()
        t6 = time.perf_counter()
        for _ in range(steps):
            alt.forward(dev["x"], dev, out=out)
        torch.cuda.synchronize()
        fp8_mfma_ms = (time.perf_counter() - t6) * 1e3 / steps
        alt.close()

    routing = layer.new_routing()                 # one extra, untimed call fetches the routing result
    layer.forward(dev["x"], dev, out=out, routing=routing)
    torch.cuda.synchronize()
    tasks0, tasks1 = layer.task_counts()
    cnt = routing["expert_count"].cpu().numpy()
    kept = int(cnt.sum())
    flops = wl.ffn_flops(c, kept)
    layer_flops = flops + 2.0 * c.tokens * c.hidden_size * c.num_experts
    ffn = stats(samples["ffn"][-steps:])
    queue = layer.ffn_mode == 2   # one launch of the task-queue kernel; otherwise one launch per projection
    fp8 = c.torch_dtype == api.DTYPE_FP8
    widened = fp8 and layer.kernel_dtype != c.torch_dtype   # the FFN stage widens the weights, then runs the bf16 tiles
    # fp32 layers: the matrix-core tile (128-row blocks) or the vector-ALU kernel (64-row blocks)
    f32_kind = "" if c.torch_dtype != api.DTYPE_F32 else ("_f32_tile" if layer.plan["block_rows"] == 128 else "_f32")
    if w.bound == "hbm" and fp8:
        active = int((cnt > 0).sum())
        nbytes = wl.fp8_ffn_bytes(c, active, kept)
        roof = {"bound": "hbm", "achieved": nbytes / (ffn["mean"] * 1e-3) / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                "kernel": "ffn_persistent_fp8_kernel" if queue else "ffn_tiled_fp8_kernel x2",
                "algorithmic_bytes": nbytes, "active_experts": active,
                # the whole step held against the same bytes: what a caller of moe_forward sees
                "layer_frac": nbytes / (ms_per_step * 1e-3) / 1e9 / PEAK_HBM_GBS}
    else:
        e4m3_mfma = fp8 and layer.options.get("fp8_mfma") == 1
        roof = {"bound": "mfma", "achieved": flops / (ffn["mean"] * 1e-3) / 1e12,
                "peak": PEAK_F32_TFLOPS if c.torch_dtype == api.DTYPE_F32 else (PEAK_FP8_TFLOPS if e4m3_mfma else PEAK_BF16_TFLOPS),
                "unit": "TFLOP/s",
                "kernel": "quant_rows128_kernel x2 + ffn_tiled_fp8_mfma_kernel x2" if e4m3_mfma else
                          (("ffn_persistent_fp8_tile_kernel" if queue else "ffn_tiled_fp8_tile_kernel x2")
                           if fp8 and not widened else
                           ("widen_block128_kernel x%d + " % (3 if c.hidden_act == api.ACT_SWIGLU else 2) if widened else "") +
                           ("ffn_persistent%s_kernel" if queue else "ffn_tiled%s_kernel x2") % f32_kind),
                "algorithmic_flops": flops}
        roof["layer_frac"] = layer_flops / (ms_per_step * 1e-3) / 1e12 / roof["peak"]
    roof["frac"] = roof["achieved"] / roof["peak"]
    roof["kernel_ms"] = ffn["mean"]
    roof["kernel_ms_median"] = ffn["median"]
    roof["kernel_ms_min"] = ffn["min"]
    plan = ""
    if fp8 and w.bound == "mfma" and not widened:
        plan = "/e4m3_mfma" if layer.options.get("fp8_mfma") == 1 else "/e4m3_tile"
    t = MEASURED_TRAFFIC.get(name + plan)
    digest = kernel_digest(t["sources"]) if t else None
    same_schedule = t is not None and t.get("ffn_mode", 2) == layer.ffn_mode
    if same_schedule and t["kernel_digest"] == digest:
        roof["traffic"] = t["bytes"]
        roof["traffic_source"] = "%s (kernel sources %s)" % (t["profile"], digest)
    else:
        roof["traffic"] = None
        roof["traffic_source"] = ("kernel sources changed since %s was collected" % t["profile"]) if same_schedule \
            else "no counter run for this kernel"
    res = {
        "workload": w.describe(), "tokens_per_s": c.tokens / (ms_per_step * 1e-3), "ms_per_step": ms_per_step,
        "ms_per_step_with_events": ms_per_step_events, "ms_per_step_graph_replay": graph_ms if graph_err is None else graph_err,
        "ms_per_step_prepared_weights": prepared_ms,
        "ms_per_step_fp8_mfma": fp8_mfma_ms,
        "step_ms": stats(step_ms), "steps": steps, "warmup": warmup,
        "tflops": layer_flops / (ms_per_step * 1e-3) / 1e12,
        "stage_ms": {k: round(v, 4) for k, v in stage_mean.items() if k != "calls"},
        "stage_ms_median": {k: round(statistics.median(v[-steps:]), 4) for k, v in samples.items()},
        "ffn_mode": layer.ffn_mode, "block_rows": layer.plan["block_rows"],
        "persistent_blocks": layer.arch["persistent_blocks"], "kept_assignments": kept, "tile_tasks": [tasks0, tasks1],
        "options": layer.options,
        # row blocks the FFN ran against the row blocks its rows would fill (the rest is padding of ragged last blocks)
        "row_blocks": int(sum((int(n) + layer.plan["block_rows"] - 1) // layer.plan["block_rows"] for n in cnt)),
        "row_blocks_full": round(kept / layer.plan["block_rows"], 2),
        # entry/exit stamps of the queue kernel's workgroups in the last call (microseconds)
        "queue_balance": {k: round(v, 1) for k, v in layer.queue_balance().items()} if queue else None,
        "roofline": roof,
    }
    return res, layer, dev, out, routing


def measure_backward(layer, cfg, dev, routing, steps, warmup):
    """Times the backward building blocks of both projections on the workload's routing: data gradients as grouped
    products with the transposed weight, weight gradients per expert.  Synthetic upstream gradients; the transposes of
    the weights are timed separately (a training step makes them once per optimizer step, not once per layer call)."""
    import torch
    import cuplayground_amd as moe
    c = cfg
    A, H, I, E = c.tokens * c.expert_top_k, c.hidden_size, c.intermediate_size, c.num_experts
    g = torch.Generator(device="cuda").manual_seed(7)
    dt = layer.act_dtype
    cnt, off = routing["expert_count"], routing["expert_offset"]
    kept = int(cnt.sum().item())
    dy = torch.randn(A, H, generator=g, device="cuda", dtype=torch.float32).to(dt)     # d loss / d y rows
    hrows = torch.randn(A, I, generator=g, device="cuda", dtype=torch.float32).to(dt)  # the saved intermediate rows
    xrows = torch.randn(A, H, generator=g, device="cuda", dtype=torch.float32).to(dt)  # the gathered token rows

    def timed(fn):
        for _ in range(warmup):
            fn()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        for a, b in ev:
            a.record(); fn(); b.record()
        torch.cuda.synchronize()
        return statistics.median(a.elapsed_time(b) for a, b in ev)

    res = {}
    w_down_t = moe.transpose(dev["w_down"])           # [E, I, H]
    w_up_t = moe.transpose(dev["w_up"])               # [E, H, I]
    res["transpose_w_down_ms"] = timed(lambda: moe.transpose(dev["w_down"], out=w_down_t))
    out_i = torch.zeros(A, I, dtype=dt, device="cuda")
    out_h = torch.zeros(A, H, dtype=dt, device="cuda")
    dw_down = torch.empty(E, H, I, dtype=dt, device="cuda")
    dw_up = torch.empty(E, I, H, dtype=dt, device="cuda")
    flops = 2.0 * kept * H * I
    ops = {
        "dgrad_down": lambda: layer.expert_gemm(dy, w_down_t, None, cnt, off, out=out_i),       # dH = dY . W_down
        "wgrad_down": lambda: layer.expert_wgrad(dy, hrows, cnt, off, out=dw_down),              # dW_down = dY^T . H
        "dgrad_up": lambda: layer.expert_gemm(hrows, w_up_t, None, cnt, off, out=out_h),         # dX = dU . W_up
        "wgrad_up": lambda: layer.expert_wgrad(hrows, xrows, cnt, off, out=dw_up),               # dW_up = dU^T . X
    }
    for name, fn in ops.items():
        ms = timed(fn)
        res[name] = {"ms": round(ms, 4), "tflops": round(flops / (ms * 1e-3) / 1e12, 1),
                     "frac": round(flops / (ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 4)}
    res["flops_per_op"] = flops
    # the activation's derivative: a pass of its own over dH (reads dH, U [, G]; writes dU [, dG]) against the same
    # arithmetic in the epilogue of the down projection's data gradient (dH never reaches memory)
    gated = c.hidden_act == moe.api.ACT_SWIGLU
    urows = hrows
    grows = hrows.clone() if gated else None
    du = torch.zeros(A, I, dtype=dt, device="cuda")
    dg = torch.zeros(A, I, dtype=dt, device="cuda") if gated else None
    res["act_backward_ms"] = round(timed(lambda: layer.act_backward(out_i, urows, grows, du=du, dg=dg)), 4)
    if layer.fused_act_backward:
        res["dgrad_down_act_fused_ms"] = round(timed(
            lambda: layer.expert_gemm_act_backward(dy, w_down_t, urows, grows, cnt, off, du=du, dg=dg)), 4)
    return res


def to_host(d):
    """Device operands -> the numpy layout the oracle takes (bf16 as uint16 bit patterns)."""
    import numpy as np
    import torch
    out = {}
    for k, v in d.items():
        if v.dtype == torch.bfloat16:
            out[k] = v.view(torch.int16).cpu().numpy().view(np.uint16)
        else:
            out[k] = v.cpu().numpy()
    return out


def task_trace_summary(layer, dev, out):
    """One more forward call with the queue kernel's per-task trace on: durations by projection and row-block fill,
    the gaps between a workgroup's consecutive tasks, and how long workgroups sit idle behind their last task."""
    import numpy as np
    import torch
    layer.enable_task_trace(1 << 17)
    layer.forward(dev["x"], dev, out=out)
    torch.cuda.synchronize()
    rec = layer.task_trace()
    layer.disable_task_trace()
    dur = rec["end_us"] - rec["start_us"]
    full = int(rec["rows"].max())
    # a task that computed one of P partial sums of its tile (option tail_split) carries 1 + 4 * part + 16 * P in `phase`
    parts = rec["phase"] >> 4
    phase = rec["phase"] & 3
    groups = []
    for ph in sorted(set(phase.tolist())):          # 0 up, 1 down projection; 2: a combine sweep of an idle workgroup (option combine = 2)
        for np_ in sorted(set(parts[phase == ph].tolist())):
            for lo, hi, label in ((full, full, "full"), (full // 2 + 1, full - 1, "more than half"), (1, full // 2, "at most half")):
                m = (phase == ph) & (parts == np_) & (rec["rows"] >= lo) & (rec["rows"] <= hi)
                if m.any():
                    g = {"phase": ph, "rows": label, "tasks": int(m.sum()), "mean_us": round(float(dur[m].mean()), 2),
                         "median_us": round(float(np.median(dur[m])), 2), "min_us": round(float(dur[m].min()), 2),
                         "max_us": round(float(dur[m].max()), 2)}
                    if np_:
                        g["partial_sums_per_tile"] = int(np_)
                    groups.append(g)
    gaps = {0: [], 1: [], 2: [], 3: []}
    busy, idle_after, per_wg = [], [], []
    end = float(rec["end_us"].max())
    for w in np.unique(rec["workgroup"]):
        r = np.sort(rec[rec["workgroup"] == w], order="start_us")
        for a, b in zip(r[:-1], r[1:]):
            gaps[int(b["phase"]) & 3].append(float(b["start_us"] - a["end_us"]))
        busy.append(float((r["end_us"] - r["start_us"]).sum()))
        idle_after.append(end - float(r["end_us"][-1]))
        per_wg.append(len(r))
    def st(v):
        return None if not v else {"mean_us": round(float(np.mean(v)), 2), "median_us": round(float(np.median(v)), 2),
                                   "max_us": round(float(np.max(v)), 2), "n": len(v)}
    return {"tasks": int(len(rec)), "block_rows": full, "span_us": round(end, 1), "by_kind": groups,
            "gap_before_up_task": st(gaps[0]), "gap_before_down_task": st(gaps[1]),
            "workgroups": len(busy), "mean_busy_us": round(float(np.mean(busy)), 1),
            "mean_idle_after_last_task_us": round(float(np.mean(idle_after)), 1),
            "max_idle_after_last_task_us": round(float(np.max(idle_after)), 1),
            "tasks_per_workgroup": [int(min(per_wg)), int(max(per_wg))],
            "note": "one extra forward call with moe_set_task_trace on (two clock reads and one atomic per task); a "
                    "down-projection task's dependency wait lies in its gap, not in its duration"}


def host_cores():
    """(threads to use, physical cores of this host): physical cores are the distinct (package, core) pairs of
    /proc/cpuinfo; the thread count is that, capped by OMP_NUM_THREADS (a GPU box hands a job its share of the host)."""
    phys = set()
    try:
        pkg = core = None
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("physical id"):
                    pkg = line.split(":")[1].strip()
                elif line.startswith("core id"):
                    core = line.split(":")[1].strip()
                elif not line.strip():
                    if core is not None:
                        phys.add((pkg, core))
                    pkg = core = None
        if core is not None:
            phys.add((pkg, core))
    except OSError:
        pass
    physical = len(phys) or (os.cpu_count() or 1)
    threads = physical
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit() and int(env) >= 1:
        threads = min(threads, int(env))
    return threads, physical


def cpu_leg(name, dev, out, routing, seconds, seed, oracle_share=0.5):
    """The CPU baseline (libtorch layer, then the oracle) on a bounded token sample, and the parity spot check of the
    GPU output against the oracle on the same sample.  The only part of this script that touches oracle/.
    `seconds` bounds the libtorch sample; the oracle gets `oracle_share` of that."""
    import numpy as np
    import torch
    from cuplayground_amd import api, workloads as wl
    from cuplayground_amd.torch_op import torch_cpu_layer
    from oracle import binding as ob

    w = wl.WORKLOADS[name]
    c = w.config
    S = c.tokens
    fp8 = c.torch_dtype == api.DTYPE_FP8
    threads, physical = host_cores()
    torch.set_num_threads(threads)
    rng = np.random.default_rng(seed)
    order = rng.permutation(S)

    # ---- libtorch CPU layer: weights widened once (bf16 -> fp32; e4m3 -> bf16) outside the timed region ----
    mats = [n for n in ("w_up", "w_gate", "w_down") if n in dev]
    host = {k: v.cpu() for k, v in dev.items() if not (fp8 and (k in mats or k.startswith("s_")))}
    if fp8:
        # the library's own inverse of the block quantiser, on the GPU (exact: bf16(e4m3 * scale)), then one copy down
        cw = {n: api.dequantize_block128(dev[n], dev["s_" + n[2:]]).cpu() for n in mats}
        prep = "e4m3 weights dequantised to bf16 once outside the timed region, bf16 linear"
    elif c.torch_dtype == api.DTYPE_BF16:
        cw = {n: host[n].float() for n in mats}
        prep = "bf16 storage, weights widened to fp32 once outside the timed region, fp32 matmul"
    else:
        cw = {n: host[n] for n in mats}
        prep = "fp32"

    def run_torch(tokens):
        import dataclasses
        sub = dataclasses.replace(c, micro_batch=1, sequence_len=len(tokens))
        xs = host["x"][torch.from_numpy(tokens.astype(np.int64))]
        t = time.perf_counter()
        o, idx = torch_cpu_layer(xs, sub, host["gate_w"], cw["w_up"], cw.get("w_gate"), cw["w_down"],
                                 host.get("gate_bias"))
        return time.perf_counter() - t, o, idx

    n0 = min(S, 64)
    dt0, _, _ = run_torch(order[:n0])                       # warm-up of the thread pool and a first estimate
    dt0, _, _ = run_torch(order[:n0])
    n = int(min(S, max(n0, seconds * n0 / max(dt0, 1e-6))))
    dt, o_cpu, idx_cpu = run_torch(order[:n])
    libtorch = {"value": n / dt, "unit": "tokens/s", "cores": threads, "host_physical_cores": physical,
                "kind": "port", "engine": "libtorch",
                "sample": "%d of %d tokens through the whole layer in libtorch CPU ops (linear, softmax/sigmoid, topk, "
                          "stable sort, index_select, per-expert linear/act/linear, index_add; %s), %.2f s on %d threads"
                          % (n, S, prep, dt, threads)}
    # the same tokens on the GPU: rows agree where the CPU router picked the same experts (its fp32 sum runs in
    # another order, so near-ties may differ) and no capacity drop depends on the rest of the batch
    sel = torch.from_numpy(order[:n].astype(np.int64))
    same = (idx_cpu == routing["topk_idx"].cpu()[sel].long()).all(dim=1).numpy()
    if not c.drop_tokens and same.any():
        g = out[sel.cuda()].float().cpu().numpy()[same]
        r = o_cpu.float().numpy()[same]
        libtorch["max_rel_err_gpu_vs_libtorch"] = float(np.abs(g - r).max() / max(np.abs(r).max(), 1e-30))
        libtorch["tokens_with_same_routing"] = int(same.sum())
    del cw, host

    # ---- the CPU oracle on (a part of) the same sample + parity of the GPU output ----
    ocfg = ob.Cfg(S=S, H=c.hidden_size, I=c.intermediate_size, E=c.num_experts, k=c.expert_top_k, act=c.hidden_act,
                  dtype=c.torch_dtype, gate_fn=c.gate_fn, norm_topk=c.norm_topk_prob, drop=c.drop_tokens,
                  capacity_factor=c.capacity_factor, zipf_bias=w.zipf_bias)
    hostnp = to_host(dev)
    r = {k: v.cpu().numpy() for k, v in routing.items()}
    tok = order.astype(np.int32)
    m0 = min(4, S)
    t = time.perf_counter()
    rows = ob.forward_tokens(ocfg, hostnp, r["topk_idx"], r["topk_w"], r["slot"], tok[:m0])
    d0 = time.perf_counter() - t
    extra = int(min(S - m0, max(0, oracle_share * seconds / max(d0 / m0, 1e-9) - m0)))
    if extra > 0:
        t = time.perf_counter()
        rows2 = ob.forward_tokens(ocfg, hostnp, r["topk_idx"], r["topk_w"], r["slot"], tok[m0:m0 + extra])
        d0 += time.perf_counter() - t
        rows = np.concatenate([rows, rows2])
        m0 += extra
    oracle = {"value": m0 / d0, "unit": "tokens/s", "cores": ob.num_threads(), "kind": "port", "engine": "oracle (C11 + OpenMP)",
              "sample": "%d of %d tokens through the oracle's expert FFN + combine (routing taken as given), %.2f s"
                        % (m0, S, d0)}
    got = out[torch.from_numpy(tok[:m0].astype(np.int64)).cuda()].float().cpu().numpy()
    ref = ob.to_f32(rows, ocfg.act_dtype)
    parity = float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))
    want = ob.route(ocfg, hostnp)
    exact = all(np.array_equal(r[k], want[k]) for k in ("topk_idx", "slot", "expert_count"))
    return libtorch, oracle, {"routing_bit_exact": exact, "max_rel_err_sample": parity, "sample_tokens": m0}


def main():
    from cuplayground_amd import workloads as wl
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="mixtral", choices=sorted(wl.WORKLOADS))
    ap.add_argument("--extra", default="decode_fp8,mid,finegrained,reference_default,prefill_fp8",
                    help="comma-separated workloads measured besides the headline one (\"\" or none: skip)")
    ap.add_argument("--extra-steps", type=int, default=20)
    ap.add_argument("--ffn-mode", type=int, default=0, help="0 auto, 1 tiled (two launches), 2 persistent queue")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample (0 = skip)")
    ap.add_argument("--extra-cpu-seconds", type=float, default=1.5,
                    help="target CPU time of the baseline sample of each --extra workload (0 = skip)")
    ap.add_argument("--option", action="append", default=[], metavar="FIELD=VALUE",
                    help="a tuning option of the handle by its moe_options field name (repeatable), e.g. --option "
                         "combine=0 --option tail_round=0; applies to every workload measured; without any, handles are "
                         "created by moe_create (library defaults, MOE355_* environment variables honoured)")
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--balanced-routing", action="store_true",
                    help="experiment: replace the router's inputs so that every expert receives exactly S*k/E rows "
                         "(no ragged last row blocks); the FFN arithmetic is unchanged")
    ap.add_argument("--backward", action="store_true",
                    help="also time the backward building blocks (data and weight gradients of both projections) on "
                         "the workload's routing; bf16 / fp16 workloads only")
    ap.add_argument("--task-trace", action="store_true",
                    help="also run one forward call with the queue kernel's per-task trace on and print its summary "
                         "(durations by projection and row-block fill, gaps, idle tails)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy (a known-size reference for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the MoE layer with all experts resident on ONE GPU; --gpus %d is not "
              "supported (no collectives, no sharding across GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    import cuplayground_amd as moe
    from cuplayground_amd import api

    torch.cuda.set_device(0)
    moe.load_library()
    main_w = wl.WORKLOADS[args.workload]
    options = None
    if args.option:
        options = {}
        for kv in args.option:
            key, _, val = kv.partition("=")
            options[key.strip()] = int(val)
    res, layer, dev, out, routing = measure(args.workload, args.steps, args.warmup, args.seed, args.ffn_mode,
                                            args.calibrate_copy, args.balanced_routing, options)
    arch = layer.arch
    # ceilings measured on this box in this run (the published peaks assume the maximum clock)
    peaks = moe.measured_peaks()
    roof = res["roofline"]
    # for the MFMA bound: the issue-only rate on random operands (the power limit lowers the clock on real data)
    if roof["bound"] == "hbm" or roof["peak"] == PEAK_BF16_TFLOPS:
        roof["measured_peak"] = peaks["hbm_read_gbs"] if roof["bound"] == "hbm" else peaks["mfma_bf16_tflops_random_operands"]
        roof["frac_of_measured_peak"] = roof["achieved"] / roof["measured_peak"]

    trace = None
    if args.task_trace and layer.ffn_mode == 2:
        trace = task_trace_summary(layer, dev, out)
    backward = None
    if args.backward:
        backward = measure_backward(layer, main_w.config, dev, routing, args.steps, args.warmup)
    cpu = cpu_oracle = parity = None
    if args.cpu_seconds > 0:
        cpu, cpu_oracle, parity = cpu_leg(args.workload, dev, out, routing, args.cpu_seconds, args.seed)
    layer.close()
    del layer, dev, out, routing
    torch.cuda.empty_cache()

    others = {}
    extra = [e for e in args.extra.split(",") if e and e != "none" and e != args.workload]
    for name in extra:
        if name not in wl.WORKLOADS:
            print("bench.py: unknown workload %r in --extra" % name, file=sys.stderr)
            sys.exit(2)
        r, l2, d2, o2, rt2 = measure(name, args.extra_steps, args.warmup, args.seed, args.ffn_mode, options=options,
                                     other_plans=True)
        if args.extra_cpu_seconds > 0:      # every workload has its CPU baseline beside it, on a smaller sample
            r["cpu_baseline"], r["cpu_baseline_oracle"], r["parity"] = cpu_leg(name, d2, o2, rt2, args.extra_cpu_seconds,
                                                                                args.seed)
        l2.close()
        del l2, d2, o2, rt2
        torch.cuda.empty_cache()
        others[name] = r

    dtype = {api.DTYPE_F32: "f32", api.DTYPE_BF16: "bf16", api.DTYPE_FP8: "fp8_e4m3_w/bf16_act"}
    line = {
        "metric": "MoE layer forward tokens/s (%s shape, 1 MI355X)" % args.workload,
        "value": res["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": res["ms_per_step"],
        # a second pass over the same steps carries the hipEvents behind step_ms, stage_ms and roofline.kernel_ms
        "ms_per_step_with_events": res["ms_per_step_with_events"], "step_ms": res["step_ms"],
        # the same steps as replays of a HIP graph that holds one forward call
        "ms_per_step_graph_replay": res["ms_per_step_graph_replay"],
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dtype[main_w.config.torch_dtype], "data": "synthetic",
        "config": {"workload": res["workload"], "ffn_mode": res["ffn_mode"], "block_rows": res["block_rows"],
                   "persistent_blocks": res["persistent_blocks"], "kept_assignments": res["kept_assignments"],
                   "tile_tasks": res["tile_tasks"], "row_blocks": res["row_blocks"],
                   "row_blocks_full": res["row_blocks_full"], "balanced_routing": bool(args.balanced_routing)},
        "queue_balance": res["queue_balance"],
        "task_trace": trace,
        "tflops": res["tflops"],
        "stage_ms": res["stage_ms"], "stage_ms_median": res["stage_ms_median"],
        "device": {"name": arch["name"], "compute_units": arch["compute_units"], "xcds": arch["xcds"],
                   "max_clock_khz": arch["max_clock_khz"],
                   "measured_mfma_bf16_tflops": round(peaks["mfma_bf16_tflops"], 1),
                   "measured_mfma_bf16_tflops_random_operands": round(peaks["mfma_bf16_tflops_random_operands"], 1),
                   "measured_hbm_read_gbs": round(peaks["hbm_read_gbs"], 1)},
        "roofline": roof, "cpu_baseline": cpu, "cpu_baseline_oracle": cpu_oracle, "parity": parity,
        "workloads": others,
    }
    if backward is not None:
        line["backward"] = backward
    print(json.dumps(line))


if __name__ == "__main__":
    main()
