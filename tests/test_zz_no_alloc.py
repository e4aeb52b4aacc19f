"""moe_forward_static: the whole layer with the workspace taken from the library's own per-GPU array (for callers
that cannot allocate).  Same kernels as moe_forward, so the two must agree bit for bit -- on two calls in a row, the
second on a smaller layer, which reuses the same array with the first call's contents still in it."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, upload_inputs

pytestmark = pytest.mark.gpu
ROUTING_KEYS = ("topk_idx", "topk_w", "slot", "expert_count", "expert_offset", "token_indices")

FIRST = ob.Cfg(S=1024, H=512, I=768, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=1, capacity_factor=1.25)
SECOND = ob.Cfg(S=96, H=256, I=128, E=16, k=4, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0)
FP8 = ob.Cfg(S=64, H=512, I=256, E=32, k=8, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0)


def _run(moe, cfg, inp, static, mode=0):
    import torch
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, allocate_workspace=not static)
    dev = upload_inputs(cfg, inp)
    routing = layer.new_routing()
    out = torch.empty(cfg.S, cfg.H, dtype=layer.act_dtype, device="cuda")
    torch.cuda.synchronize()
    # the property the entry point exists for: with out and routing preallocated, the call takes no device memory --
    # neither from the driver nor from torch's allocator
    free0, reserved0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_reserved()
    layer.forward(dev["x"], dev, out=out, routing=routing, static_workspace=static)
    torch.cuda.synchronize()
    if static:
        assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_reserved() == reserved0
        t0, t1 = layer.task_counts()             # read from the static array (the layer owns no workspace)
        assert t0 > 0 and t1 > 0
        if layer.ffn_mode == 2:
            assert layer.queue_balance()["workgroups"] > 0
    res = {k: from_device(v) for k, v in routing.items()}
    res["out"] = from_device(out)
    layer.close()
    return res


def test_static_workspace_forward_matches_moe_forward():
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    import cuplayground_amd as moe
    moe.load_library()
    for cfg, seed, mode in ((FIRST, 21, 2), (SECOND, 22, 0), (FP8, 23, 2), (FIRST, 24, 1)):
        inp = ob.make_inputs(cfg, seed=seed)
        want = _run(moe, cfg, inp, static=False, mode=mode)
        got = _run(moe, cfg, inp, static=True, mode=mode)
        for key in ROUTING_KEYS:
            assert np.array_equal(got[key], want[key]), (cfg, key)
        assert np.array_equal(got["out"], want["out"]), cfg            # same kernels: bit for bit
        ref = ob.forward(cfg, inp)                                       # and right, not merely equal
        for key in ("topk_idx", "slot", "expert_count"):
            assert np.array_equal(got[key], ref[key]), (cfg, key)
        err = max_rel_err(ob.to_f32(got["out"], cfg.act_dtype), ob.to_f32(ref["out"], cfg.act_dtype))
        assert err <= OUT_TOL[cfg.dtype], err


def test_static_workspace_rejects_a_layer_that_does_not_fit():
    import torch
    import cuplayground_amd as moe
    big = ob.Cfg(S=8192, H=1024, I=2048, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0)
    pc = product_config(big)
    assert pc.workspace_bytes() > 32 << 20
    layer = moe.MoELayer(pc, allocate_workspace=False)
    bf = dict(dtype=torch.bfloat16, device="cuda")
    w = dict(gate_w=torch.zeros(big.E, big.H, **bf), w_up=torch.zeros(big.E, big.I, big.H, **bf),
             w_gate=torch.zeros(big.E, big.I, big.H, **bf), w_down=torch.zeros(big.E, big.H, big.I, **bf))
    with pytest.raises(moe.MoEError) as e:
        layer.forward(torch.zeros(big.S, big.H, **bf), w, static_workspace=True)
    assert e.value.status == 3   # MOE_ERR_WORKSPACE: a clear error, nothing enqueued
    layer.close()
