#!/usr/bin/env python3
"""Benchmark of the fused MoE forward on one MI355X.

A step is one moe_forward call (gate -> slots -> expert FFN -> combine) on one batch of synthetic tokens already
resident in HBM.  Default workload: the Mixtral-shape configuration (S=8192, H=4096, I=14336, E=8, top-2, SwiGLU,
bf16, dropless).  Prints one JSON line:
  value      tokens/s of the whole layer
  roofline   the expert-FFN kernel (the dominant launch) against the bf16 MFMA peak -- or the HBM peak for the fp8
             decode shape -- from hipEvents recorded around that kernel inside the timed steps
  cpu_baseline  the CPU oracle (a port: the reference's own CPU hook, torching.cuh:8-11, is empty) timed on a
             bounded token sample of the same workload on this box's host cores
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0     # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0         # MI355X HBM3E
# Bytes per FFN-kernel launch that crossed the L2 <-> memory-fabric boundary, from two rocprofv3 --pmc runs of this
# script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter showed for a 1 GiB
# device copy in the same run (--calibrate-copy): read x2.000, write x1.000.  Summaries are kept under profiles/.
MEASURED_TRAFFIC_BYTES = {"mixtral": 19.130e9 + 0.631e9, "decode_fp8": 9.924e9 + 0.013e9}


def workloads():
    from oracle import binding as ob
    return {"mixtral": ("C3", ob.BASELINE["C3"]), "mid": ("C2", ob.BASELINE["C2"]),
            "finegrained": ("C4", ob.BASELINE["C4"]), "decode_fp8": ("C5", ob.BASELINE["C5"]),
            "tiny": ("C1", ob.BASELINE["C1"])}


def make_device_inputs(cfg, seed):
    """Synthetic operands generated on the GPU: tokens N(0,1), weights N(0,0.02), rounded to storage."""
    import torch
    import cuplayground_amd as moe
    from oracle import binding as ob
    g = torch.Generator(device="cuda").manual_seed(seed)
    adt = torch.float32 if cfg.dtype == ob.F32 else torch.bfloat16
    S, H, I, E = cfg.S, cfg.H, cfg.I, cfg.E

    def normal(shape, std, dtype):
        out = torch.empty(shape, dtype=dtype, device="cuda")
        n0 = shape[0]
        for i in range(n0):            # expert by expert: bounds the fp32 temporary
            out[i] = (torch.randn(shape[1:], generator=g, device="cuda", dtype=torch.float32) * std).to(dtype)
        return out

    d = {"x": (torch.randn(S, H, generator=g, device="cuda", dtype=torch.float32)).to(adt),
         "gate_w": (torch.randn(E, H, generator=g, device="cuda", dtype=torch.float32) * 0.02).to(adt)}
    if cfg.zipf_bias:
        d["gate_bias"] = torch.from_numpy(ob.zipf_gate_bias(E, seed)).cuda()
    names = ["w_up", "w_down"] + (["w_gate"] if cfg.act == ob.ACT_SWIGLU else [])
    for n in names:
        shape = (E, H, I) if n == "w_down" else (E, I, H)
        if cfg.dtype == ob.FP8:
            w = normal(shape, 0.02, torch.float32)
            d[n], d["s_" + n[2:]] = moe.quantize_block128(w)   # e4m3 codes + one scale per 128x128 block
            del w
        else:
            d[n] = normal(shape, 0.02, adt)
    return d


def to_host(cfg, d):
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


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="mixtral", choices=sorted(workloads()))
    ap.add_argument("--ffn-mode", type=int, default=0, help="0 auto, 1 tiled (two launches), 2 persistent queue")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample (0 = skip)")
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 1 GiB device-to-device copy (a known-size reference for HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs the MoE layer with all experts resident on ONE GPU; --gpus %d is not "
              "supported (no collectives, no sharding across GPUs)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import cuplayground_amd as moe
    from oracle import binding as ob

    tag, cfg = workloads()[args.workload]
    torch.cuda.set_device(0)
    moe.load_library()
    pc = moe.MoEConfig(capacity_factor=cfg.capacity_factor, drop_tokens=cfg.drop, expert_top_k=cfg.k,
                       hidden_act=cfg.act, hidden_size=cfg.H, intermediate_size=cfg.I, micro_batch=1,
                       num_experts=cfg.E, sequence_len=cfg.S, torch_dtype=cfg.dtype, gate_fn=cfg.gate_fn,
                       norm_topk_prob=cfg.norm_topk)
    layer = moe.MoELayer(pc, ffn_mode=args.ffn_mode)
    dev = make_device_inputs(cfg, args.seed)
    routing = layer.new_routing()
    out = torch.empty(cfg.S, cfg.H, dtype=layer.act_dtype, device="cuda")

    if args.calibrate_copy:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)              # reads 1 GiB and writes 1 GiB
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        layer.forward(dev["x"], dev, out=out, routing=routing)
    torch.cuda.synchronize()
    layer.set_stage_timing(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        layer.forward(dev["x"], dev, out=out, routing=routing)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    stage = layer.stage_ms()
    layer.set_stage_timing(False)
    tasks0, tasks1 = layer.task_counts()
    ms_per_step = (t1 - t0) * 1e3 / args.steps

    cnt = routing["expert_count"].cpu().numpy()
    kept = int(cnt.sum())
    g = 3 if cfg.act == ob.ACT_SWIGLU else 2
    ffn_flops = 2.0 * g * kept * cfg.H * cfg.I
    layer_flops = ffn_flops + 2.0 * cfg.S * cfg.H * cfg.E
    ffn_s = stage["ffn"] * 1e-3
    queue = layer.ffn_mode == 2   # one launch of the task-queue kernel; otherwise one launch per projection
    if cfg.dtype == ob.FP8:
        active = int((cnt > 0).sum())
        scale_bytes = 3 * (cfg.H // 128) * (cfg.I // 128) * 4
        ffn_bytes = active * (3.0 * cfg.H * cfg.I + scale_bytes) + 2.0 * kept * cfg.H * 2
        roofline = {"bound": "hbm", "achieved": ffn_bytes / ffn_s / 1e9, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "traffic": None, "kernel": "ffn_persistent_fp8_kernel" if queue else "ffn_tiled_fp8_kernel x2", "kernel_ms": stage["ffn"],
                    "algorithmic_bytes": ffn_bytes, "active_experts": active}
    else:
        roofline = {"bound": "mfma", "achieved": ffn_flops / ffn_s / 1e12, "peak": PEAK_BF16_TFLOPS,
                    "unit": "TFLOP/s", "traffic": None, "kernel": "ffn_persistent_kernel" if queue else "ffn_tiled_kernel x2", "kernel_ms": stage["ffn"],
                    "algorithmic_flops": ffn_flops}
        if cfg.dtype == ob.F32:
            roofline["peak"] = 157.3
    roofline["frac"] = roofline["achieved"] / roofline["peak"]
    roofline["traffic"] = MEASURED_TRAFFIC_BYTES.get(args.workload) if queue else None
    # ceilings measured on this box in this run (the published peaks assume the maximum clock)
    peaks = moe.measured_peaks()
    arch = layer.arch
    # for the MFMA bound: the issue-only rate on random operands (the power limit lowers the clock on real data)
    roofline["measured_peak"] = peaks["hbm_read_gbs"] if cfg.dtype == ob.FP8 else peaks["mfma_bf16_tflops_random_operands"]
    roofline["frac_of_measured_peak"] = roofline["achieved"] / roofline["measured_peak"]

    # ---- CPU baseline + parity spot check on the same sample ----
    cpu = None
    parity = None
    if args.cpu_seconds > 0:
        host = to_host(cfg, dev)
        r = {k: v.cpu().numpy() for k, v in routing.items()}
        rng = np.random.default_rng(args.seed)
        order = rng.permutation(cfg.S).astype(np.int32)
        n = min(4, cfg.S)
        t = time.perf_counter()
        rows = ob.forward_tokens(cfg, host, r["topk_idx"], r["topk_w"], r["slot"], order[:n])
        dt = time.perf_counter() - t
        extra = int(min(cfg.S - n, max(0, args.cpu_seconds / max(dt / n, 1e-9) - n)))
        if extra > 0:
            t = time.perf_counter()
            rows2 = ob.forward_tokens(cfg, host, r["topk_idx"], r["topk_w"], r["slot"], order[n:n + extra])
            dt += time.perf_counter() - t
            rows = np.concatenate([rows, rows2])
            n += extra
        cpu = {"value": n / dt, "unit": "tokens/s", "cores": ob.num_threads(), "kind": "port",
               "sample": "%d of %d tokens through the CPU oracle's expert FFN + combine (routing taken as given), "
                         "%.1f s" % (n, cfg.S, dt)}
        got = out[torch.from_numpy(order[:n].astype(np.int64)).cuda()]
        got = got.float().cpu().numpy()
        ref = ob.to_f32(rows, cfg.act_dtype)
        parity = float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))
        want = ob.route(cfg, host)
        routing_exact = all(np.array_equal(r[k], want[k]) for k in ("topk_idx", "slot", "expert_count"))
    else:
        routing_exact = None

    line = {
        "metric": "MoE layer forward tokens/s (%s shape, 1 MI355X)" % args.workload,
        "value": cfg.S / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": {ob.F32: "f32", ob.BF16: "bf16", ob.FP8: "fp8_e4m3_w/bf16_act"}[cfg.dtype],
        "data": "synthetic",
        "config": {"workload": "%s: S=%d H=%d I=%d E=%d top%d %s %s" % (
            tag, cfg.S, cfg.H, cfg.I, cfg.E, cfg.k, {0: "relu", 1: "gelu", 2: "swiglu"}[cfg.act],
            "drop cf=%g" % cfg.capacity_factor if cfg.drop else "dropless"),
            "ffn_mode": layer.ffn_mode, "persistent_blocks": layer.arch["persistent_blocks"], "kept_assignments": kept, "tile_tasks": [tasks0, tasks1]},
        "tflops": layer_flops / (ms_per_step * 1e-3) / 1e12,
        "stage_ms": {k: round(v, 4) for k, v in stage.items()},
        "device": {"name": arch["name"], "compute_units": arch["compute_units"], "max_clock_khz": arch["max_clock_khz"],
                   "measured_mfma_bf16_tflops": round(peaks["mfma_bf16_tflops"], 1),
                   "measured_mfma_bf16_tflops_random_operands": round(peaks["mfma_bf16_tflops_random_operands"], 1),
                   "measured_hbm_read_gbs": round(peaks["hbm_read_gbs"], 1)},
        "roofline": roofline, "cpu_baseline": cpu,
        "parity": {"routing_bit_exact": routing_exact, "max_rel_err_sample": parity},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
