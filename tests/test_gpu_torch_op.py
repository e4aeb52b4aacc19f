"""torch.ops.moe355.forward (the PyTorch operator over the C ABI) against the CPU oracle and a plain-torch layer."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, as_f32, from_device, max_rel_err, product_config, upload_inputs

pytestmark = pytest.mark.gpu

OP_CASES = {
    "bf16_swiglu_top2": ob.Cfg(S=256, H=128, I=256, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0),
    "bf16_gelu_drop": ob.Cfg(S=384, H=256, I=128, E=4, k=2, act=ob.ACT_GELU, dtype=ob.BF16, drop=1, capacity_factor=1.0),
    "f32_relu_top1": ob.Cfg(S=128, H=64, I=128, E=4, k=1, act=ob.ACT_RELU, dtype=ob.F32, norm_topk=0, drop=0),
    "fp8_swiglu_sigmoid": ob.Cfg(S=64, H=256, I=256, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID,
                                 drop=0),
}


@pytest.fixture(scope="module")
def top():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import cuplayground_amd.torch_op as top
    return top


def call_op(cfg, dev):
    import torch
    return torch.ops.moe355.forward(dev["x"], dev["gate_w"], dev["w_up"], dev.get("w_gate"), dev["w_down"],
                                    product_config(cfg).to_json(), dev.get("gate_bias"), dev.get("b_up"),
                                    dev.get("b_gate"), dev.get("b_down"), dev.get("s_up"), dev.get("s_gate"),
                                    dev.get("s_down"))


@pytest.mark.parametrize("name", sorted(OP_CASES))
def test_operator_vs_oracle(top, name):
    import torch
    cfg = OP_CASES[name]
    inp = ob.make_inputs(cfg, seed=23)
    want = ob.forward(cfg, inp)
    dev = upload_inputs(cfg, inp)
    out = call_op(cfg, dev)
    out2 = call_op(cfg, dev)                       # second call reuses the cached handle and workspace
    torch.cuda.synchronize()
    got = as_f32(from_device(out), cfg.dtype)
    assert max_rel_err(got, as_f32(want["out"], cfg.dtype)) <= OUT_TOL[cfg.dtype]
    assert torch.equal(out, out2)


@pytest.mark.parametrize("name", ["bf16_swiglu_top2", "bf16_gelu_drop", "f32_relu_top1"])
def test_operator_vs_plain_torch_layer(top, name):
    """Same routing (taken from the oracle) fed to the plain-torch layer: the two FFN + combine paths must agree."""
    import torch
    cfg = OP_CASES[name]
    inp = ob.make_inputs(cfg, seed=29)
    want = ob.forward(cfg, inp)
    dev = upload_inputs(cfg, inp)
    out = call_op(cfg, dev)
    topk = (torch.from_numpy(want["topk_idx"]).cuda(), torch.from_numpy(want["topk_w"]).cuda())
    ref = top.torch_reference(dev["x"], product_config(cfg), dev["gate_w"], dev["w_up"], dev.get("w_gate"),
                              dev["w_down"], topk=topk)
    torch.cuda.synchronize()
    tol = 2e-5 if cfg.dtype == ob.F32 else OUT_TOL[cfg.dtype]   # torch's fp32 GEMM sums in another order
    assert max_rel_err(out.float().cpu().numpy(), ref.float().cpu().numpy()) <= tol
    # and with its own router the plain-torch layer picks the same experts on this seed
    ref_own = top.torch_reference(dev["x"], product_config(cfg), dev["gate_w"], dev["w_up"], dev.get("w_gate"),
                                  dev["w_down"])
    assert max_rel_err(out.float().cpu().numpy(), ref_own.float().cpu().numpy()) <= tol


def test_module_wrapper_and_meta(top):
    import torch
    from cuplayground_amd import MoEConfig
    cfg = MoEConfig(expert_top_k=2, hidden_act=2, hidden_size=128, intermediate_size=256, micro_batch=2,
                    num_experts=8, sequence_len=128, torch_dtype=2, norm_topk_prob=1)
    layer = top.MoE355(cfg, seed=3)
    x = torch.randn(256, 128, device="cuda", generator=torch.Generator(device="cuda").manual_seed(5)).bfloat16()
    with torch.no_grad():
        y = layer(x)
        ref = layer.reference(x)
    assert y.shape == (256, 128) and y.dtype == torch.bfloat16
    assert max_rel_err(y.float().cpu().numpy(), ref.float().cpu().numpy()) <= OUT_TOL[ob.BF16]
    m = torch.ops.moe355.forward(x.to("meta"), layer.gate_w.to("meta"), layer.w_up.to("meta"), layer.w_gate.to("meta"),
                                 layer.w_down.to("meta"), layer.config_json)
    assert m.shape == x.shape and m.device.type == "meta"


def test_operator_rejects_bad_arguments(top):
    import torch
    cfg = OP_CASES["bf16_swiglu_top2"]
    dev = upload_inputs(cfg, ob.make_inputs(cfg, seed=1))
    bad = dict(dev)
    bad["x"] = dev["x"][:-1]
    with pytest.raises(ValueError):
        call_op(cfg, bad)
    bad = dict(dev)
    bad["w_gate"] = None
    with pytest.raises(ValueError):
        call_op(cfg, bad)
    bad = dict(dev)
    bad["w_up"] = dev["w_up"].transpose(1, 2)
    with pytest.raises(ValueError):
        call_op(cfg, bad)
