"""The BASELINE configurations at full size on the GPU.

The oracle cannot run a whole 5.8 TFLOP layer in test time, so: routing (integers) is compared in full, the
layer output on a seeded sample of tokens, and the rest through properties that hold at any size (the two
independent FFN schedules agree bit for bit, fully dropped tokens are exactly zero, kept rows add up)."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, upload_inputs

pytestmark = pytest.mark.gpu
FFN_TILED, FFN_PERSISTENT = 1, 2
SAMPLE = {"C2": 48, "C3": 16, "C4": 48, "C5": 24}


@pytest.mark.parametrize("name", ["C2", "C3", "C4", "C5"])
def test_baseline_config_full_size(name):
    import torch
    import cuplayground_amd as moe
    assert torch.cuda.is_available()
    cfg = ob.BASELINE[name]
    print("config", name, cfg, flush=True)
    inp = ob.make_inputs(cfg, seed=42)
    want = ob.route(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT)
    dev = upload_inputs(cfg, inp)
    routing = layer.new_routing()
    out = layer.forward(dev["x"], dev, routing=routing)
    torch.cuda.synchronize()
    t0, t1 = layer.task_counts()
    got = {k: from_device(v) for k, v in routing.items()}
    for key in ("topk_idx", "slot", "expert_count", "expert_offset", "token_indices"):
        assert np.array_equal(got[key], want[key]), key
    assert np.abs(got["topk_w"] - want["topk_w"]).max() <= 2e-6
    kept = int(want["expert_count"].sum())
    assert kept == int((want["slot"] >= 0).sum())
    if not cfg.drop:
        assert kept == cfg.S * cfg.k
    assert t0 > 0 and t1 > 0

    # sampled output parity: tokens drawn with a fixed seed, always including a dropped-pair token if any
    rng = np.random.default_rng(7)
    tokens = rng.choice(cfg.S, size=SAMPLE[name], replace=False).astype(np.int32)
    partly = np.nonzero((want["slot"] < 0).any(axis=1))[0]
    if partly.size:
        tokens[0] = partly[0]
    ref = ob.to_f32(ob.forward_tokens(cfg, inp, want["topk_idx"], want["topk_w"], want["slot"], tokens), cfg.act_dtype)
    o = out.float().cpu().numpy()
    err = max_rel_err(o[tokens], ref)
    print(name, "sampled max rel err", err, flush=True)
    assert err <= OUT_TOL[cfg.dtype], err

    dead = (want["slot"] < 0).all(axis=1)
    assert (o[dead] == 0).all()
    assert np.isfinite(o).all()

    # the two-launch schedule shares no queue state with the persistent one and must agree bit for bit
    layer.set_ffn_mode(FFN_TILED)
    out2 = layer.forward(dev["x"], dev)
    assert torch.equal(out, out2)
    layer.close()
