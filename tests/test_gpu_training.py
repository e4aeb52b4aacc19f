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


@pytest.mark.parametrize("act,dtype,drop", [(2, 2, 0), (1, 2, 1), (0, 3, 0), (2, 3, 1)])
def test_trainable_layer_matches_torch_autograd(moe, act, dtype, drop):
    import torch
    from cuplayground_amd import training, torch_op
    cfg = moe.MoEConfig(capacity_factor=1.0, drop_tokens=drop, expert_top_k=2, hidden_act=act, hidden_size=256,
                        intermediate_size=384 if act == 2 else 512, micro_batch=1, num_experts=6, sequence_len=700,
                        torch_dtype=dtype, gate_fn=0, norm_topk_prob=1, is_training=1)
    m = training.MoE355Train(cfg, init_std=0.05, seed=3)
    g = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(cfg.tokens, cfg.hidden_size, generator=g, device="cuda").to(m.layer.act_dtype).requires_grad_(True)
    dout = torch.randn(cfg.tokens, cfg.hidden_size, generator=g, device="cuda").to(m.layer.act_dtype)
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

    assert rel(out.float(), ref) <= (1e-2 if dtype == 2 else 2e-3)
    tol = 2e-2 if dtype == 2 else 4e-3      # gradients pass through two rounded products
    assert rel(x.grad.float(), xr.grad) <= tol
    for n, p in m.named_parameters():
        assert p.grad is not None and torch.isfinite(p.grad.float()).all(), n
        assert rel(p.grad.float(), ps[n].grad) <= tol, n
    if drop:                                # some pairs were dropped in this configuration: the test covers that path
        assert int((m.route(x)[1]["pair_row"] < 0).sum()) > 0


def test_fp32_layers_are_refused(moe):
    from cuplayground_amd import training
    with pytest.raises(ValueError):
        training.MoE355Train(moe.MoEConfig(hidden_size=64, intermediate_size=64, micro_batch=1, sequence_len=128))


@pytest.mark.parametrize("act", [1, 2])
def test_backward_chain_through_the_c_abi_matches_torch_autograd(moe, act):
    """A whole expert-FFN backward composed of the library's entry points only (combine backward, weight and data
    gradients, activation backward; torch only gathers rows and scatters them back), against torch autograd on the
    fp32 layer with the same routing and fixed gate weights."""
    import torch
    from cuplayground_amd import api, torch_op
    cfg = moe.MoEConfig(capacity_factor=1.0, drop_tokens=1, expert_top_k=2, hidden_act=act, hidden_size=256,
                        intermediate_size=384 if act == 2 else 512, micro_batch=1, num_experts=5, sequence_len=600,
                        torch_dtype=2, gate_fn=0, norm_topk_prob=1, is_training=1)
    layer = moe.MoELayer(cfg)
    g = torch.Generator(device="cuda").manual_seed(5)
    dt = torch.bfloat16
    S, H, I, E = cfg.tokens, cfg.hidden_size, cfg.intermediate_size, cfg.num_experts
    rnd = lambda *s, std=1.0: (torch.randn(*s, generator=g, device="cuda") * std).to(dt)
    x, gate_w = rnd(S, H), rnd(E, H, std=0.05)
    w_up, w_down = rnd(E, I, H, std=0.05), rnd(E, H, I, std=0.05)
    w_gate = rnd(E, I, H, std=0.05) if act == 2 else None
    dout = rnd(S, H)
    idx, w = layer.gate(x, gate_w)
    r = layer.route(idx)
    cnt, off, rows = r["expert_count"], r["expert_offset"], r["pair_row"]
    # forward, keeping what the backward needs
    x_rows = x.index_select(0, r["token_indices"].clamp(min=0).long())
    u = layer.expert_gemm(x_rows, w_up, None, cnt, off)
    gg = layer.expert_gemm(x_rows, w_gate, None, cnt, off) if act == 2 else None
    h = (torch.nn.functional.silu(gg.float()) * u.float() if act == 2 else torch.nn.functional.gelu(u.float())).to(dt)
    y = layer.expert_gemm(h, w_down, None, cnt, off)
    out = moe.combine(y, rows, w)
    # backward through the C ABI
    dy, dw_gate = layer.combine_backward(dout, y, rows, w)
    dW_down = layer.expert_wgrad(dy, h, cnt, off)
    dh = layer.expert_gemm(dy, api.transpose(w_down), None, cnt, off)
    du, dg = layer.act_backward(dh, u, gg)
    dW_up = layer.expert_wgrad(du, x_rows, cnt, off)
    dx_rows = layer.expert_gemm(du, api.transpose(w_up), None, cnt, off).float()
    if act == 2:
        dW_gate = layer.expert_wgrad(dg, x_rows, cnt, off)
        dx_rows = dx_rows + layer.expert_gemm(dg, api.transpose(w_gate), None, cnt, off).float()
    kept = int(cnt.sum())
    dx = torch.zeros(S, H, device="cuda").index_add_(0, r["token_indices"][:kept].long(), dx_rows[:kept])
    # reference: fp32 parameters, torch autograd, the same routing and gate weights (held constant)
    leaf = lambda t: None if t is None else t.float().requires_grad_(True)
    xr, up_r, gate_r, down_r, w_r = leaf(x), leaf(w_up), leaf(w_gate), leaf(w_down), leaf(w)
    ref = torch_op.torch_reference(xr, cfg, gate_w.float(), up_r, gate_r, down_r, topk=(idx, w_r))
    ref.backward(dout.float())
    assert rel(out.float(), ref) <= 1e-2
    tol = 2e-2
    assert rel(dx, xr.grad) <= tol
    assert rel(dW_up.float(), up_r.grad) <= tol and rel(dW_down.float(), down_r.grad) <= tol
    if act == 2:
        assert rel(dW_gate.float(), gate_r.grad) <= tol
    assert rel(dw_gate, w_r.grad) <= tol                       # d loss / d (gate weight of each kept pair)
    assert int((rows < 0).sum()) > 0
