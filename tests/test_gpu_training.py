"""The trainable layer built on the backward building blocks, against the same layer written in torch ops with fp32
parameters and torch's own autograd (forward values and every gradient)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def moe():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import cuplayground_amd
    cuplayground_amd.load_library()
    return cuplayground_amd


def rel(a, b):
    a, b = a.detach().double(), b.detach().double()
    return float((a - b).abs().max() / b.abs().max().clamp(min=1e-30))


@pytest.mark.parametrize("act,dtype,drop,inter", [(2, 2, 0, 384), (1, 2, 1, 512), (0, 3, 0, 512), (2, 3, 1, 384), (0, 0, 0, 512),
                                                  (2, 0, 1, 384), (1, 1, 0, 512), (2, 2, 1, 512), (2, 3, 0, 512)])
def test_trainable_layer_matches_torch_autograd(moe, act, dtype, drop, inter):
    import torch
    from cuplayground_amd import training, torch_op
    cfg = moe.MoEConfig(capacity_factor=1.0, drop_tokens=drop, expert_top_k=2, hidden_act=act, hidden_size=256,
                        intermediate_size=inter, micro_batch=1, num_experts=6, sequence_len=700,
                        torch_dtype=dtype, gate_fn=0, norm_topk_prob=1, is_training=1)
    m = training.MoE355Train(cfg, init_std=0.05, seed=3)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(cfg.tokens, cfg.hidden_size, generator=g, device="cuda").to(m.layer.act_dtype).requires_grad_(True)
    dout = torch.randn(cfg.tokens, cfg.hidden_size, generator=g, device="cuda").to(m.layer.act_dtype)
    # the activation's derivative rides in the epilogue of the down projection's data gradient where the layer has
    # that kernel (16-bit, 256 | intermediate size), else the two building blocks run one after the other
    assert m.layer.fused_act_backward == (dtype in (2, 3) and inter % 256 == 0)
    out = m(x)
    out.backward(dout)

    # the same layer in torch ops on fp32 copies of the same (16-bit valued) parameters, routing taken from the library
    idx, _ = m.route(x)
    xr = x.detach().float().requires_grad_(True)
    ps = {n: p.detach().float().requires_grad_(True) for n, p in m.named_parameters()}
    logits = xr @ ps["gate_w"].t()
    w = torch.softmax(logits, 1).gather(1, idx.long())
    w = w / w.sum(1, keepdim=True)
    ref = torch_op.torch_reference(xr, cfg, ps["gate_w"], ps["w_up"], ps.get("w_gate"), ps["w_down"], topk=(idx, w))
    ref.backward(dout.float())

    assert rel(out.float(), ref) <= {2: 1e-2, 3: 2e-3}.get(dtype, 2e-5)
    tol = {2: 2e-2, 3: 4e-3}.get(dtype, 1e-4)      # 16-bit gradients pass through two rounded products; fp32: summation order
    assert rel(x.grad.float(), xr.grad) <= tol
    for n, p in m.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad.float()).all(), n
        assert rel(p.grad.float(), ps[n].grad) <= tol, n
    if drop:                                # some pairs were dropped in this configuration: the test covers that path
        assert int((m.route(x)[1]["pair_row"] < 0).sum()) > 0


def test_e4m3_layers_are_refused(moe):
    from cuplayground_amd import training
    with pytest.raises(ValueError):
        training.MoE355Train(moe.MoEConfig(hidden_size=128, intermediate_size=128, micro_batch=1, sequence_len=128,
                                           torch_dtype=4))
