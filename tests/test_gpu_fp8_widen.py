"""e4m3-weight layers with very many rows per expert: the weights are widened to bf16 in the workspace (csrc/quant.hip)
and the layer runs the bf16 tile GEMM.  The widening against the oracle's decode to the bit, the layer against the
oracle, against the e4m3 tile GEMM, and bit for bit against a bf16 layer on the widened weights."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, to_device, upload_inputs
from test_gpu_layer import FFN_PERSISTENT, FFN_TILED, check_routing

pytestmark = pytest.mark.gpu

SHAPES = {
    # 256-row blocks with ragged tails, SwiGLU, three scale blocks along K of the down projection
    "swiglu": ob.Cfg(S=1100, H=256, I=384, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SOFTMAX, drop=0),
    # two weight matrices per expert, biases, capacity drops
    "gelu_bias": ob.Cfg(S=900, H=384, I=256, E=5, k=2, act=ob.ACT_GELU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=1,
                        capacity_factor=1.25),
}


def _forward(cfg, dev, mode, widen):
    import torch
    import cuplayground_amd as moe
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode,
                         options={} if widen is None else {"fp8_widen": widen, "fp8_mfma": 0})
    routing = layer.new_routing()
    out = torch.full((cfg.S, cfg.H), float("nan"), dtype=layer.act_dtype, device="cuda")
    for _ in range(2):   # the workspace copy of the weights is rewritten by every call
        layer.forward(dev["x"], dev, out=out, routing=routing)
    torch.cuda.synchronize()
    layer.task_counts()
    res = {k: from_device(v) for k, v in routing.items()}
    res["bits"] = from_device(out)
    res["out"] = ob.to_f32(res["bits"], cfg.act_dtype)
    res["workspace_bytes"] = layer.workspace_bytes
    layer.close()
    return res


def test_widening_is_the_oracle_decode_rounded_once():
    import torch
    import cuplayground_amd as moe
    assert torch.cuda.is_available(), "these tests need the MI355X"
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((3, 256, 384)) * np.exp(rng.uniform(-8, 8, (3, 256, 1)))).astype(np.float32)
    w[1, :128, 128:256] = 0.0        # an all-zero block: scale 1
    q, s = ob.quant_block128(w)
    q[2, 5, :254] = np.arange(254, dtype=np.uint8) + (np.arange(254) >= 127)   # every finite code point once
    want = ob.f32_to_bf16(ob.dequant_block128(q, s))
    got = from_device(moe.dequantize_block128(to_device(q, "u8"), to_device(s, "f32")))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
@pytest.mark.parametrize("name", sorted(SHAPES))
def test_widened_layer(name, mode):
    import cuplayground_amd as moe
    cfg = SHAPES[name]
    inp = ob.make_inputs(cfg, seed=37, with_bias="bias" in name)
    want = ob.forward(cfg, inp)
    dev = upload_inputs(cfg, inp)
    got = _forward(cfg, dev, mode, 1)
    check_routing(got, want)
    assert max_rel_err(got["out"], ob.to_f32(want["out"], cfg.act_dtype)) <= OUT_TOL[ob.FP8]
    assert not got["out"][(want["slot"] < 0).all(axis=1)].any()
    # the e4m3 tile GEMM scales fp32 partial sums instead of rounding scaled weights to bf16
    tile = _forward(cfg, dev, mode, 0)
    assert max_rel_err(got["out"], tile["out"]) <= 1e-2
    assert got["workspace_bytes"] - tile["workspace_bytes"] >= (3 if cfg.act == ob.ACT_SWIGLU else 2) * cfg.E * cfg.H * cfg.I * 2
    # a bf16 layer handed the widened weights computes exactly the same thing
    wide = dict(dev)
    for n in ("up", "gate", "down"):
        if "w_" + n in dev:
            wide["w_" + n] = moe.dequantize_block128(dev["w_" + n], dev["s_" + n])
            del wide["s_" + n]
    bf = _forward(cfg.scaled(dtype=ob.BF16), wide, mode, None)
    assert np.array_equal(got["bits"], bf["bits"])


def test_plan_widens_from_a_thousand_rows_per_expert():
    import cuplayground_amd as moe
    mid = moe.MoELayer(product_config(ob.Cfg(S=1024, H=256, I=256, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8)), options={})
    big = moe.MoELayer(product_config(ob.Cfg(S=2048, H=256, I=256, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8)), options={})
    assert mid.plan["block_rows"] == 128
    # the workspace grows by the bf16 copies of the three weight matrices, not only by the rows of twice the tokens
    rows = 2 * (2048 - 1024) * (256 + 256) * 2
    assert big.workspace_bytes - mid.workspace_bytes >= 3 * 4 * 256 * 256 * 2 + rows
    mid.close(); big.close()


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
def test_prepared_weights_change_no_bit_and_save_the_workspace(mode, tmp_path):
    """moe_prepare_weights writes the bf16 copies once; a forward call that carries them skips the widening launches and
    must reproduce the per-call result bit for bit.  A handle created with prepared_weights = 1 asks for a workspace
    without the copies and refuses a call that comes without them.  The prepared form survives a trip through a
    packed-layer file."""
    import torch
    import cuplayground_amd as moe
    from cuplayground_amd import weights as wts
    cfg = SHAPES["swiglu"]
    inp = ob.make_inputs(cfg, seed=41)
    dev = upload_inputs(cfg, inp)
    per_call = _forward(cfg, dev, mode, 1)

    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, options={"fp8_widen": 1, "fp8_mfma": 0, "prepared_weights": 1})
    assert layer.options["prepared_weights"] == 1
    assert layer.prepared_bytes == 3 * cfg.E * cfg.H * cfg.I * 2
    assert per_call["workspace_bytes"] - layer.workspace_bytes >= layer.prepared_bytes
    with pytest.raises(moe.MoEError) as e:
        layer.forward(dev["x"], dev)                     # promised prepared weights, none given
    assert e.value.status == 4
    packed = wts.prepare_packed(dev_weights(dev), layer)
    assert packed["prepared"].numel() == layer.prepared_bytes
    # the prepared operands are exactly the library's own dequantisation of the three matrices: up, down, gate
    want = torch.cat([moe.dequantize_block128(dev["w_" + n], dev["s_" + n]).reshape(-1) for n in ("up", "down", "gate")])
    assert torch.equal(packed["prepared"].view(torch.bfloat16), want)
    path = str(tmp_path / "layer.safetensors")
    wts.save_packed(path, packed, product_config(cfg))
    loaded, pc = wts.load_packed(path)
    assert pc == product_config(cfg) and torch.equal(loaded["prepared"], packed["prepared"])
    out = torch.full((cfg.S, cfg.H), float("nan"), dtype=layer.act_dtype, device="cuda")
    for _ in range(2):
        layer.forward(dev["x"], dict(loaded, x=dev["x"]), out=out)
    torch.cuda.synchronize()
    layer.task_counts()
    assert np.array_equal(from_device(out), per_call["bits"])
    layer.close()

    # a handle that keeps the copies in its workspace takes prepared weights too; a plan that prepares nothing has none
    plain = moe.MoELayer(product_config(cfg), ffn_mode=mode, options={"fp8_widen": 1, "fp8_mfma": 0})
    out2 = plain.forward(dev["x"], dict(loaded, x=dev["x"]))
    torch.cuda.synchronize()
    assert np.array_equal(from_device(out2), per_call["bits"])
    plain.close()
    tile = moe.MoELayer(product_config(cfg), ffn_mode=mode, options={"fp8_widen": 0, "fp8_mfma": 0})
    assert tile.prepared_bytes == 0 and tile.prepare_weights(dev) is None
    with pytest.raises(moe.MoEError):
        tile.forward(dev["x"], dict(loaded, x=dev["x"]))   # prepared operands of another plan
    tile.close()


def dev_weights(dev):
    return {k: v for k, v in dev.items() if k != "x"}
