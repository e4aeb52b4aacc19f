"""Down-projection tiles of the last row blocks computed as partial sums (option tail_split; csrc/ffn_bf16.hip:
partial_tile_arrive and the summing epilogue, csrc/queue_order.hpp: split_tail).  The result must depend on the number of
parts only, never on the schedule: the task queue and the two launches agree bit for bit, repeated calls agree bit for
bit; against the oracle the layer keeps its tolerance, and against whole tiles it differs by the rounding of a
differently associated fp32 sum only."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, upload_inputs
from test_gpu_layer import FFN_PERSISTENT, FFN_TILED, check_routing

pytestmark = pytest.mark.gpu

SHAPES = {
    # every row block is in the tail (few blocks): ragged last blocks, an expert that may stay empty, biases
    "small_gelu_bias": (ob.Cfg(S=700, H=512, I=512, E=5, k=2, act=ob.ACT_GELU, dtype=ob.BF16, gate_fn=ob.GATE_SOFTMAX, drop=0), True),
    # SwiGLU, fp16, capacity drops
    "small_swiglu_f16": (ob.Cfg(S=900, H=256, I=1024, E=3, k=2, act=ob.ACT_SWIGLU, dtype=ob.F16, gate_fn=ob.GATE_SIGMOID, drop=1,
                                capacity_factor=1.25), False),
    # more row blocks than the tail holds: the run of one expert is cut where the partial sums begin
    "cut": (ob.Cfg(S=6144, H=2048, I=512, E=6, k=2, act=ob.ACT_RELU, dtype=ob.BF16, gate_fn=ob.GATE_SOFTMAX, drop=0), False),
}


def _forward(cfg, dev, mode, options, calls=2):
    import torch
    import cuplayground_amd as moe
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, options=options)
    routing = layer.new_routing()
    out = torch.full((cfg.S, cfg.H), float("nan"), dtype=layer.act_dtype, device="cuda")
    bits = []
    for _ in range(calls):
        layer.forward(dev["x"], dev, out=out, routing=routing)
        torch.cuda.synchronize()
        bits.append(from_device(out).copy())
    layer.task_counts()                     # raises if a dependency wait expired
    res = {k: from_device(v) for k, v in routing.items()}
    res["bits"] = bits
    res["out"] = ob.to_f32(bits[-1], cfg.act_dtype)
    res["options"] = layer.options
    res["workspace_bytes"] = layer.workspace_bytes
    layer.close()
    return res


@pytest.mark.parametrize("parts", [2, 4])
@pytest.mark.parametrize("tile", [1, 2, 3])
@pytest.mark.parametrize("name", sorted(SHAPES))
def test_partial_sums_do_not_depend_on_the_schedule(name, tile, parts):
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    cfg, bias = SHAPES[name]
    inp = ob.make_inputs(cfg, seed=11, with_bias=bias)
    want = ob.forward(cfg, inp)
    dev = upload_inputs(cfg, inp)
    opts = {"tile16": tile, "tail_split": parts}
    queue = _forward(cfg, dev, FFN_PERSISTENT, opts)
    assert queue["options"]["tail_split"] == parts and queue["options"]["tile16"] == tile
    check_routing(queue, want)
    assert np.array_equal(queue["bits"][0], queue["bits"][1])
    assert max_rel_err(queue["out"], ob.to_f32(want["out"], cfg.act_dtype)) <= OUT_TOL[cfg.dtype]
    assert not queue["out"][(want["slot"] < 0).all(axis=1)].any()
    tiled = _forward(cfg, dev, FFN_TILED, opts)
    assert np.array_equal(tiled["bits"][0], tiled["bits"][1])
    assert np.array_equal(queue["bits"][1], tiled["bits"][1])
    whole = _forward(cfg, dev, FFN_PERSISTENT, {"tile16": tile, "tail_split": 1}, calls=1)
    assert whole["options"]["tail_split"] == 1
    assert whole["workspace_bytes"] < queue["workspace_bytes"]
    # the same products, added in another order in fp32, rounded to 16 bits once: a few results move by one step of the
    # 16-bit format (bf16: 2^-8 of the value at most)
    assert max_rel_err(queue["out"], whole["out"]) <= 2.0 ** -8
    assert (queue["bits"][1] != whole["bits"][0]).mean() < 0.2


def test_option_is_ignored_where_it_does_not_apply():
    import cuplayground_amd as moe
    base = ob.Cfg(S=512, H=512, I=512, E=4, k=2, act=ob.ACT_GELU, dtype=ob.BF16, gate_fn=ob.GATE_SOFTMAX, drop=0)
    cases = [
        (base.scaled(I=768), {"tile16": 1, "tail_split": 4}, 1),      # 768 / 4 = 192: not a multiple of 128 per part ...
        (base.scaled(I=768), {"tile16": 1, "tail_split": 2}, 2),      # ... 768 / 2 = 384 is
        (base.scaled(I=256), {"tile16": 1, "tail_split": 4}, 1),
        (base, {"tile16": 0, "tail_split": 2}, 1),                    # the 128 x 128 tile has no such epilogue
        (base, {"tile16": 1, "tail_split": 2, "combine": 2}, 1),      # the combine inside the kernel counts whole tiles
        (base, {"tile16": 1, "tail_split": 2, "queue_early": 1}, 1),
    ]
    for cfg, opts, want in cases:
        layer = moe.MoELayer(product_config(cfg), options=opts)
        assert layer.options["tail_split"] == want, (cfg.I, opts)
        layer.close()
    f32 = moe.MoELayer(product_config(base.scaled(dtype=ob.F32)), options={"tail_split": 2})
    assert f32.options["tail_split"] == moe.api.OPT_AUTO
    f32.close()


def test_a_part_whose_rows_never_came_hands_on_nan():
    """Every dependency wait expires at once (spin limit < 0): a part of a tile stores NaN in place of its sums, the tile
    is NaN, the stall is reported, and every kernel exits normally."""
    import torch
    import cuplayground_amd as moe
    cfg, bias = SHAPES["small_gelu_bias"]
    inp = ob.make_inputs(cfg, seed=3, with_bias=bias)
    dev = upload_inputs(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT, options={"tile16": 1, "tail_split": 2})
    layer.set_spin_limit(-1)
    out = torch.zeros((cfg.S, cfg.H), dtype=layer.act_dtype, device="cuda")
    layer.forward(dev["x"], dev, out=out)
    torch.cuda.synchronize()
    assert layer.stalled
    got = ob.to_f32(from_device(out), cfg.act_dtype)
    want = ob.forward(cfg, inp)
    routed = (want["slot"] >= 0).any(axis=1)
    assert routed.any() and np.isnan(got[routed]).all()
    layer.clear_stall()
    layer.set_spin_limit(0)
    layer.forward(dev["x"], dev, out=out)
    torch.cuda.synchronize()
    assert not layer.stalled
    assert max_rel_err(ob.to_f32(from_device(out), cfg.act_dtype), ob.to_f32(want["out"], cfg.act_dtype)) <= OUT_TOL[cfg.dtype]
    layer.close()
