"""fp32 (and tf32) layers with enough rows per expert: the 128 x 128 matrix-core tile (csrc/ffn_f32_tile.hip) against the
CPU oracle, against the vector-ALU kernel on the same inputs, and across its schedules."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, upload_inputs
from test_gpu_layer import FFN_PERSISTENT, FFN_TILED, check_routing

pytestmark = pytest.mark.gpu

SHAPES = {
    # the reference's own knob file at a fifth of its tokens: one expert, top-1, ReLU, full blocks and a ragged last one
    "reference_like": ob.Cfg(S=1700, H=256, I=512, E=1, k=1, act=ob.ACT_RELU, dtype=ob.F32, norm_topk=0, drop=0),
    # SwiGLU pairs, several experts with ragged tails
    "swiglu": ob.Cfg(S=700, H=256, I=384, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.F32, gate_fn=ob.GATE_SIGMOID, drop=0),
    # biases, capacity drops, experts with a handful of rows next to experts with several blocks
    "gelu_skew_drop_bias": ob.Cfg(S=1500, H=384, I=256, E=12, k=3, act=ob.ACT_GELU, dtype=ob.F32, drop=1,
                                  capacity_factor=1.0, zipf_bias=True),
    # shortest K (four slabs) in the up projection, tf32 storage type
    "tf32_short_k": ob.Cfg(S=256, H=128, I=512, E=1, k=1, act=ob.ACT_SWIGLU, dtype=ob.TF32, norm_topk=0, drop=0),
    # fewer rows than one block everywhere (the tile forced onto a small layer)
    "tiny_rows_bias": ob.Cfg(S=40, H=256, I=128, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.F32, gate_fn=ob.GATE_SIGMOID, drop=0),
}


def _run(cfg, inp, mode, tile, calls=1, combine=0):
    import torch
    import cuplayground_amd as moe
    assert torch.cuda.is_available(), "these tests need the MI355X"
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, options={"f32_tile": tile, "combine": combine})
    assert layer.plan["block_rows"] == (128 if tile else 64)
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
def test_tile_vs_oracle_and_vector_kernel(name, mode):
    cfg = SHAPES[name]
    inp = ob.make_inputs(cfg, seed=23, with_bias="bias" in name)
    want = ob.forward(cfg, inp)
    ref = ob.to_f32(want["out"], cfg.act_dtype)
    got = _run(cfg, inp, mode, 1, calls=2)
    check_routing(got, want)
    assert not np.isnan(got["out"]).any()
    assert max_rel_err(got["out"], ref) <= OUT_TOL[ob.F32]
    assert not got["out"][(want["slot"] < 0).all(axis=1)].any()
    vec = _run(cfg, inp, mode, 0)      # the same fp32 sums in another order
    assert max_rel_err(got["out"], vec["out"]) <= OUT_TOL[ob.F32]


@pytest.mark.parametrize("name", sorted(SHAPES))
def test_tile_schedules_agree_bit_for_bit(name):
    cfg = SHAPES[name]
    inp = ob.make_inputs(cfg, seed=31, with_bias="bias" in name)
    a = _run(cfg, inp, FFN_TILED, 1)
    b = _run(cfg, inp, FFN_PERSISTENT, 1)
    assert np.array_equal(a["out"], b["out"])
    for combine in (1, 2):      # inside the FFN kernels: by arrival counters, as tasks of the queue
        c = _run(cfg, inp, FFN_PERSISTENT, 1, combine=combine)
        assert np.array_equal(a["out"], c["out"]), combine


def test_plan_follows_rows_per_expert_and_shape():
    import cuplayground_amd as moe
    small = moe.MoELayer(product_config(ob.BASELINE["C1"]), options={})                # 16 rows per expert
    few_tiles = moe.MoELayer(product_config(ob.Cfg(S=1024, H=256, I=512, E=8, k=1, act=ob.ACT_GELU, dtype=ob.F32)), options={})
    ragged = moe.MoELayer(product_config(ob.Cfg(S=8192, H=960, I=4096, E=1, k=1, act=ob.ACT_RELU, dtype=ob.F32)), options={})
    big = moe.MoELayer(product_config(ob.Cfg(S=8192, H=1024, I=4096, E=1, k=1, act=ob.ACT_RELU, dtype=ob.F32)), options={})
    assert [l.plan["block_rows"] for l in (small, few_tiles, ragged, big)] == [64, 64, 64, 128]
    assert big.plan["col_tiles_up"] == 4096 // 128 and big.plan["col_tiles_down"] == 1024 // 128
    for l in (small, few_tiles, ragged, big):
        l.close()
