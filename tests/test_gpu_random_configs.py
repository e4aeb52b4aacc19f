"""Seeded random layer shapes crossed with the tuning knobs (tile, FFN mode, queue count, early start of the next
task, combine inside the FFN kernels, task order inside a queue segment, e4m3 streamer or tile): every combination must match the CPU oracle -- routing bit for bit, output
within the dtype's bound -- because no knob is allowed to change what is computed (tail_split alone re-associates a sum,
within the same bound).  Where the layer has the fused data gradient of the down projection, it is checked against
the two calls it replaces on the same routing."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, to_device, upload_inputs
from test_gpu_layer import check_routing

pytestmark = pytest.mark.gpu


def _cases(n=36, seed=2024):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        dtype = [ob.BF16, ob.BF16, ob.F16, ob.F32, ob.FP8][i % 5]
        act = int(rng.choice([ob.ACT_RELU, ob.ACT_GELU, ob.ACT_SWIGLU]))
        if dtype == ob.FP8 and i % 2 == 0:
            act = ob.ACT_SWIGLU                  # e4m3 layers: SwiGLU at least every other time
        E = int(rng.choice([1, 2, 3, 4, 6, 8, 16, 40]))
        k = int(rng.integers(1, min(E, 4) + 1))
        mult = 128 if dtype == ob.FP8 else (256 if i % 2 == 0 else 64)        # multiples of 256 reach the hand-ordered tiles
        H = mult * int(rng.integers(1, 3))
        I = mult * int(rng.integers(1, 4))
        S = int(rng.integers(1, 2600 if i % 2 == 0 else 900))     # the larger ones give experts several row blocks
        drop = int(rng.integers(0, 2))
        cfg = ob.Cfg(S=S, H=H, I=I, E=E, k=k, act=act, dtype=dtype, drop=drop,
                     capacity_factor=float(rng.choice([0.5, 1.0, 1.5])), norm_topk=int(k > 1),
                     gate_fn=ob.GATE_SIGMOID if dtype == ob.FP8 else int(rng.integers(0, 2)), zipf_bias=bool(i % 3 == 0))
        knobs = dict(tile16=int(rng.integers(0, 4)), queue_groups=int(rng.choice([1, 2, 8])),
                     queue_early=int(rng.integers(0, 2)), combine=int(rng.integers(0, 2)))
        if knobs["combine"] and i % 3 == 2:
            knobs["combine"] = 2              # the combine as tasks of the FFN queue instead of by arrival counters
        knobs["row_chunk"] = i % 4            # order of the tasks inside a queue segment (0: plain; drawn outside the seeded stream)
        knobs["fp8_tile"] = i // 5 % 2        # e4m3 layers: weight streamer or tile GEMM
        knobs["gate_mfma"] = i // 2 % 2       # 16-bit layers with H % 512 = 0: logits on the vector ALU or on the matrix cores
        knobs["f32_tile"] = i // 5 % 2        # fp32 layers: vector-ALU kernel or (shape permitting) the matrix-core tile
        knobs["fp8_widen"] = i // 10 % 2      # ... or the bf16 tiles on weights widened in the workspace
        knobs["fp8_mfma"] = 0                 # bf16 tokens: the arithmetic the oracle's layer restates
        knobs["gate_fused_topk"] = i // 3 % 2 # top-k inside the logits kernel or as a launch of its own
        knobs["tail_round"] = i // 4 % 2      # the last up-projection segment moved so that the tail fills whole rounds
        # the last down-projection tiles as partial sums: re-associates an fp32 sum (other bits, the same tolerance); ignored
        # where it does not apply (the 128 x 128 tile, an intermediate size that does not divide, combine inside the
        # kernels, queue_early)
        knobs["tail_split"] = (1, 2, 4)[i // 2 % 3]
        if dtype in (ob.BF16, ob.F16) and mult == 256 and i % 4 == 0:     # ... and these cases make sure that it does apply
            knobs.update(combine=0, queue_early=0, tile16=1 + i // 4 % 3, tail_split=4 if I % 512 == 0 else 2)
        out.append(pytest.param(cfg, knobs, int(rng.integers(1, 3)), bool(rng.integers(0, 2)), id="case%02d" % i))
    return out


@pytest.mark.parametrize("cfg,knobs,mode,with_bias", _cases())
def test_random_shape_and_knobs_vs_oracle(cfg, knobs, mode, with_bias):
    import torch
    import cuplayground_amd as moe
    assert torch.cuda.is_available(), "these tests need the MI355X"
    inp = ob.make_inputs(cfg, seed=17, with_bias=with_bias)
    want = ob.forward(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, options=knobs)
    dev = upload_inputs(cfg, inp)
    routing = layer.new_routing()
    out = torch.full((cfg.S, cfg.H), float("nan"), dtype=layer.act_dtype, device="cuda")
    for _ in range(2):                       # the second call reuses every counter and table of the first
        layer.forward(dev["x"], dev, out=out, routing=routing)
    torch.cuda.synchronize()
    layer.task_counts()
    got = {k: from_device(v) for k, v in routing.items()}
    check_routing(got, want)
    o = ob.to_f32(from_device(out), cfg.act_dtype)
    ref = ob.to_f32(want["out"], cfg.act_dtype)
    assert not np.isnan(o).any()
    assert max_rel_err(o, ref) <= OUT_TOL[cfg.dtype], (knobs, mode)
    dead = (want["slot"] < 0).all(axis=1)
    assert not o[dead].any()
    if cfg.dtype in (ob.BF16, ob.F16) and layer.fused_act_backward:
        _fused_backward_is_the_chain(moe, layer, cfg, dev, routing, got)
    layer.close()


def _fused_backward_is_the_chain(moe, layer, cfg, dev, routing, got):
    """On the routing the layer just produced: the data gradient of the down projection with the activation's derivative
    in its epilogue against the two calls it replaces, bit for bit on the kept rows."""
    import torch
    kind = "bf16" if cfg.dtype == ob.BF16 else "f16"
    rng = np.random.default_rng(cfg.S + cfg.I)
    R, kept = cfg.S * cfg.k, int(got["expert_count"].sum())
    rand = lambda cols, scale: to_device(ob.from_f32(rng.standard_normal((R, cols)).astype(np.float32) * scale, cfg.dtype), kind)
    dy, u = rand(cfg.H, 1.0), rand(cfg.I, 2.0)
    g = rand(cfg.I, 2.0) if cfg.act == ob.ACT_SWIGLU else None
    cnt, off = routing["expert_count"], routing["expert_offset"]
    w_t = moe.transpose(dev["w_down"])
    du, dg = layer.expert_gemm_act_backward(dy, w_t, u, g, cnt, off)
    dh = layer.expert_gemm(dy, w_t, None, cnt, off, ob.ACT_NONE)
    du2, dg2 = layer.act_backward(dh[:kept], u[:kept], None if g is None else g[:kept])
    torch.cuda.synchronize()
    assert np.array_equal(from_device(du)[:kept], from_device(du2))
    assert not from_device(du)[kept:].any()
    if g is not None:
        assert np.array_equal(from_device(dg)[:kept], from_device(dg2))
