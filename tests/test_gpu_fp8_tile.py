"""e4m3-weight layers with many rows per expert: the 128 x 128 tile GEMM (csrc/ffn_fp8_tile.hip) against the CPU
oracle, against the weight streamer on the same inputs, and across its two schedules."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, upload_inputs
from test_gpu_layer import FFN_PERSISTENT, FFN_TILED, check_routing

pytestmark = pytest.mark.gpu

SHAPES = {
    # full blocks and a ragged last block per expert, two k blocks up / three down
    "few_experts": ob.Cfg(S=700, H=256, I=384, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0),
    # capacity drops, biases, experts with a handful of rows next to experts with several blocks
    "skew_drop_bias": ob.Cfg(S=1500, H=384, I=256, E=12, k=3, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SOFTMAX,
                             drop=1, capacity_factor=1.0, zipf_bias=True),
    # shortest K (one k block) in the up projection, one expert, exactly full blocks
    "one_expert_short_k": ob.Cfg(S=256, H=128, I=512, E=1, k=1, act=ob.ACT_SWIGLU, dtype=ob.FP8, norm_topk=0, drop=0),
    # many experts just above the plan's threshold: every row block is a partial one (about 40 of 128 rows), top-1
    "many_partial_blocks": ob.Cfg(S=2000, H=256, I=256, E=48, k=1, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SOFTMAX,
                                  norm_topk=0, drop=0),
    # up projection without SwiGLU: 128 rows of w_up per tile, activation in the epilogue; with and without biases
    "gelu_bias": ob.Cfg(S=900, H=256, I=384, E=5, k=2, act=ob.ACT_GELU, dtype=ob.FP8, gate_fn=ob.GATE_SOFTMAX, drop=1,
                        capacity_factor=1.25),
    "relu": ob.Cfg(S=640, H=384, I=128, E=3, k=1, act=ob.ACT_RELU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, norm_topk=0,
                   drop=0),
    # fewer rows than one block everywhere (the tile forced onto a decode-sized layer)
    "tiny_rows": ob.Cfg(S=40, H=256, I=128, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0),
}


def _run(cfg, inp, mode, tile, calls=1, combine=0):
    import torch
    import cuplayground_amd as moe
    assert torch.cuda.is_available(), "these tests need the MI355X"
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode,
                         options={"fp8_tile": tile, "fp8_widen": 0, "fp8_mfma": 0, "combine": combine})
    assert layer.plan["block_rows"] == (128 if tile else 16)
    dev = upload_inputs(cfg, inp)
    routing = layer.new_routing()
    out = torch.full((cfg.S, cfg.H), float("nan"), dtype=layer.act_dtype, device="cuda")
    for _ in range(calls):
        layer.forward(dev["x"], dev, out=out, routing=routing)
    torch.cuda.synchronize()
    layer.task_counts()
    res = {k: from_device(v) for k, v in routing.items()}
    res["out"] = ob.to_f32(from_device(out), cfg.act_dtype)
    layer.close()
    return res


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
@pytest.mark.parametrize("name", sorted(SHAPES))
def test_tile_gemm_vs_oracle_and_streamer(name, mode):
    cfg = SHAPES[name]
    inp = ob.make_inputs(cfg, seed=29, with_bias="bias" in name)
    want = ob.forward(cfg, inp)
    ref = ob.to_f32(want["out"], cfg.act_dtype)
    got = _run(cfg, inp, mode, 1, calls=2)
    check_routing(got, want)
    assert not np.isnan(got["out"]).any()
    assert max_rel_err(got["out"], ref) <= OUT_TOL[ob.FP8]
    assert not got["out"][(want["slot"] < 0).all(axis=1)].any()
    # the streamer computes the same block-scaled sums in another order: both round h and y to bf16 once
    stream = _run(cfg, inp, mode, 0)
    assert max_rel_err(got["out"], stream["out"]) <= 1e-2


@pytest.mark.parametrize("name", sorted(SHAPES))
def test_tile_gemm_schedules_agree_bit_for_bit(name):
    cfg = SHAPES[name]
    inp = ob.make_inputs(cfg, seed=31, with_bias="bias" in name)
    a = _run(cfg, inp, FFN_TILED, 1)
    b = _run(cfg, inp, FFN_PERSISTENT, 1)
    assert np.array_equal(a["out"], b["out"])
    for combine in (1, 2):      # inside the FFN kernels: by arrival counters, as tasks of the queue
        c = _run(cfg, inp, FFN_PERSISTENT, 1, combine=combine)
        assert np.array_equal(a["out"], c["out"]), combine


def test_plan_follows_rows_per_expert():
    """Decode-sized layers keep the weight streamer, prefill-sized ones take the tile."""
    import cuplayground_amd as moe
    small = moe.MoELayer(product_config(ob.Cfg(S=64, H=256, I=256, E=32, k=8, act=ob.ACT_SWIGLU, dtype=ob.FP8)), options={})
    big = moe.MoELayer(product_config(ob.Cfg(S=2048, H=256, I=256, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8)), options={})
    assert small.plan["block_rows"] == 16 and big.plan["block_rows"] == 128
    assert big.plan["col_tiles_up"] == 256 // 64 and big.plan["col_tiles_down"] == 256 // 128
    small.close(); big.close()


def test_prefill_sized_layer_on_a_stratified_sample():
    """A layer big enough to fill the queue kernel several times over (8 experts of about 1024 rows, 72 row blocks x
    104 column tiles): routing in full, the output on each expert's first row, tail block and block boundaries plus
    random tokens, and the two schedules bit for bit."""
    import torch
    import cuplayground_amd as moe
    from test_gpu_fullsize import stratified_tokens
    cfg = ob.Cfg(S=4096, H=2048, I=5632, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SOFTMAX, drop=0)
    inp = ob.make_inputs(cfg, seed=42)
    want = ob.route(cfg, inp)
    # fp8_widen 0: this many rows per expert would run the bf16 tile on widened weights
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT, options={"fp8_widen": 0, "fp8_mfma": 0})
    assert layer.plan["block_rows"] == 128
    dev = upload_inputs(cfg, inp)
    routing = layer.new_routing()
    out = layer.forward(dev["x"], dev, routing=routing)
    torch.cuda.synchronize()
    layer.task_counts()
    check_routing({k: from_device(v) for k, v in routing.items()}, want)
    chosen, strata, rng = stratified_tokens(cfg, want, 128)
    tokens = np.unique(np.concatenate([chosen, rng.choice(cfg.S, size=192, replace=False)])).astype(np.int32)
    print("strata", len(strata), "tokens checked", tokens.size, flush=True)
    ref = ob.to_f32(ob.forward_tokens(cfg, inp, want["topk_idx"], want["topk_w"], want["slot"], tokens), cfg.act_dtype)
    o = out.float().cpu().numpy()
    err = max_rel_err(o[tokens], ref)
    print("sampled max rel err", err, flush=True)
    assert err <= OUT_TOL[ob.FP8], err
    assert np.isfinite(o).all()
    layer.set_ffn_mode(FFN_TILED)
    out2 = layer.forward(dev["x"], dev)
    assert torch.equal(out, out2)
    layer.close()
