"""The per-task trace of the queue kernels (moe_set_task_trace / moe_get_task_trace): one record per task, each tile
exactly once, and the dependency between the projections visible in the clock stamps."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import product_config, upload_inputs
from test_gpu_layer import FFN_PERSISTENT, FFN_TILED

pytestmark = pytest.mark.gpu

CASES = {
    "bf16_large_tile": ob.Cfg(S=2500, H=256, I=512, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0),
    "bf16_small_tile": ob.Cfg(S=700, H=192, I=320, E=5, k=2, act=ob.ACT_GELU, dtype=ob.BF16, drop=1, capacity_factor=1.1),
    "f32": ob.Cfg(S=333, H=192, I=320, E=7, k=3, act=ob.ACT_SWIGLU, dtype=ob.F32, drop=1, capacity_factor=0.75),
    "f32_tile": ob.Cfg(S=900, H=256, I=384, E=3, k=2, act=ob.ACT_GELU, dtype=ob.F32, drop=0),
    "fp8_streamer": ob.Cfg(S=64, H=512, I=256, E=32, k=8, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0),
    "fp8_tile": ob.Cfg(S=1500, H=384, I=256, E=6, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0),
}


@pytest.mark.parametrize("name", sorted(CASES) + ["bf16_large_tile_early_start"])
def test_every_task_is_recorded_once_and_in_dependency_order(name):
    import torch
    import cuplayground_amd as moe
    assert torch.cuda.is_available(), "these tests need the MI355X"
    options = {}
    if name.endswith("_early_start"):        # the queue loop that starts the next task under the current tile's end
        options["queue_early"] = 1
        name = name[:-len("_early_start")]
    cfg = CASES[name]
    options["f32_tile"] = 1 if name == "f32_tile" else 0
    inp = ob.make_inputs(cfg, seed=13)
    want = ob.route(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT, options=options)
    dev = upload_inputs(cfg, inp)
    plan = layer.plan
    layer.enable_task_trace(1 << 14)
    ref = layer.forward(dev["x"], dev).clone()
    for _ in range(2):                       # the trace holds the last call only
        out = layer.forward(dev["x"], dev)
    torch.cuda.synchronize()
    t0, t1 = layer.task_counts()
    rec = layer.task_trace()
    assert len(rec) == t0 + t1
    assert (rec["phase"] == 0).sum() == t0 and (rec["phase"] == 1).sum() == t1
    keys = set(zip(rec["phase"].tolist(), rec["row_block"].tolist(), rec["col_tile"].tolist()))
    assert len(keys) == len(rec), "a tile was run twice"
    # the row blocks are the oracle's: expert-major, block_rows rows each, a shorter last one
    blocks = [(e, min(plan["block_rows"], int(c) - r0)) for e, c in enumerate(want["expert_count"])
              for r0 in range(0, int(c), plan["block_rows"])]
    for r in rec:
        assert (int(r["expert"]), int(r["rows"])) == blocks[int(r["row_block"])]
        assert 0 <= r["col_tile"] < (plan["col_tiles_down"] if r["phase"] else plan["col_tiles_up"])
    assert (rec["end_us"] >= rec["start_us"]).all() and rec["start_us"].min() == 0
    # a down-projection tile starts only after every up-projection tile of its row block has ended
    done0 = {}
    for r in rec[rec["phase"] == 0]:
        done0[int(r["row_block"])] = max(done0.get(int(r["row_block"]), 0.0), float(r["end_us"]))
    for r in rec[rec["phase"] == 1]:
        assert float(r["start_us"]) >= done0[int(r["row_block"])] - 0.011     # one tick of the 100 MHz clock
    assert torch.equal(out, ref)             # tracing changes no result
    # off again: the next call leaves the old records alone and the handle says so
    layer.disable_task_trace()
    layer.forward(dev["x"], dev)
    torch.cuda.synchronize()
    with pytest.raises(moe.MoEError):
        layer.task_trace()
    layer.close()


def test_a_short_buffer_counts_what_it_cannot_hold():
    import torch
    import cuplayground_amd as moe
    cfg = CASES["bf16_small_tile"]
    inp = ob.make_inputs(cfg, seed=13)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT)
    dev = upload_inputs(cfg, inp)
    layer.enable_task_trace(5)
    layer.forward(dev["x"], dev)
    torch.cuda.synchronize()
    t0, t1 = layer.task_counts()
    assert t0 + t1 > 5
    rec = layer.task_trace()
    assert len(rec) == 5 and len({(int(r["phase"]), int(r["row_block"]), int(r["col_tile"])) for r in rec}) == 5
    layer.close()


def test_two_launch_mode_leaves_no_records():
    import torch
    import cuplayground_amd as moe
    cfg = CASES["bf16_small_tile"]
    inp = ob.make_inputs(cfg, seed=13)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_TILED)
    dev = upload_inputs(cfg, inp)
    layer.enable_task_trace(64)
    layer.forward(dev["x"], dev)
    torch.cuda.synchronize()
    assert len(layer.task_trace()) == 0
    layer.close()
