"""A trainable MoE layer over the backward building blocks of libmoe355 (fp32, tf32, bf16 and fp16 layers).

The reference declares a training knob (`is_training`, aristos_config.schema.json:20-23) that none of its code reads.
Here it has a consumer: `MoE355Train` runs the expert projections through `moe_expert_gemm` and gets their gradients
from `moe_expert_gemm` on the transposed weight (data gradient) and `moe_expert_wgrad` (weight gradient).  Routing
decisions (top-k indices, slots, capacity drops) come from the library's router and are not differentiated; the gate
weights that scale the expert outputs are recomputed in torch from the same logits formula, so the router's weight
matrix and the tokens receive gradients through them.  The activation and the down projection are one autograd node
(`_ActDown`): its backward is `moe_expert_gemm_act_backward` -- the data gradient of the down projection with the
activation's derivative in the product's epilogue -- where the layer has it, else `moe_expert_gemm` followed by
`moe_act_backward`.  Gather and the weighted combine are indexing work left to torch's autograd.  There is no CPU path:
every tensor lives on the GPU.
"""
from __future__ import annotations

import torch

from . import api


class _ExpertLinear(torch.autograd.Function):
    """rows[r] -> rows[r] . w[e(r)]^T over packed expert-major rows (rows of no expert give zeros)."""

    @staticmethod
    def forward(ctx, a_rows, w, layer, count, offset):
        a_rows = a_rows.contiguous()
        ctx.save_for_backward(a_rows, w, count, offset)
        ctx.layer = layer
        return layer.expert_gemm(a_rows, w, None, count, offset, api.ACT_NONE)

    @staticmethod
    def backward(ctx, dy):
        a_rows, w, count, offset = ctx.saved_tensors
        layer = ctx.layer
        dy = dy.contiguous()
        da = dw = None
        if ctx.needs_input_grad[0]:
            da = layer.expert_gemm(dy, api.transpose(w), None, count, offset, api.ACT_NONE)      # dA = dY . W
        if ctx.needs_input_grad[1]:
            dw = layer.expert_wgrad(dy, a_rows, count, offset)                                     # dW[e] = dY_e^T . A_e
        return da, dw, None, None, None


def expert_linear(a_rows, w, layer: api.MoELayer, expert_count, expert_offset):
    return _ExpertLinear.apply(a_rows, w, layer, expert_count, expert_offset)


class _ActDown(torch.autograd.Function):
    """(u rows, g rows or None) -> act(u, g) . w_down[e(r)]^T over packed expert-major rows."""

    @staticmethod
    def forward(ctx, u, g, w, layer, count, offset):
        act = layer.cfg.hidden_act
        if act == api.ACT_SWIGLU:
            h = torch.nn.functional.silu(g.float()) * u.float()
        elif act == api.ACT_GELU:
            h = torch.nn.functional.gelu(u.float())
        else:
            h = torch.relu(u.float())
        h = h.to(u.dtype)
        ctx.save_for_backward(u, g, h, w, count, offset)
        ctx.layer = layer
        return layer.expert_gemm(h, w, None, count, offset, api.ACT_NONE)

    @staticmethod
    def backward(ctx, dy):
        u, g, h, w, count, offset = ctx.saved_tensors
        layer = ctx.layer
        dy = dy.contiguous()
        w_t = api.transpose(w)                                                                     # [E, I, H]
        if layer.fused_act_backward:
            du, dg = layer.expert_gemm_act_backward(dy, w_t, u, g, count, offset)
        else:
            dh = layer.expert_gemm(dy, w_t, None, count, offset, api.ACT_NONE)                     # dH = dY . W_down
            du, dg = layer.act_backward(dh, u, g)
        dw = layer.expert_wgrad(dy, h, count, offset) if ctx.needs_input_grad[2] else None
        return du, dg, dw, None, None, None


def act_down(u_rows, g_rows, w_down, layer: api.MoELayer, expert_count, expert_offset):
    return _ActDown.apply(u_rows.contiguous(), None if g_rows is None else g_rows.contiguous(), w_down, layer,
                          expert_count, expert_offset)


class MoE355Train(torch.nn.Module):
    """forward(x [S,H]) -> [S,H] with gradients for x, gate_w, w_up, w_gate and w_down."""

    def __init__(self, cfg: api.MoEConfig, init_std: float = 0.02, seed: int = 0):
        super().__init__()
        if cfg.torch_dtype == api.DTYPE_FP8:
            raise ValueError("the backward building blocks exist for fp32, tf32, bf16 and fp16 layers, not for e4m3 weights")
        self.cfg = cfg
        self.layer = api.MoELayer(cfg)
        dt = self.layer.act_dtype
        E, H, I = cfg.num_experts, cfg.hidden_size, cfg.intermediate_size
        g = torch.Generator(device="cpu").manual_seed(seed)

        def p(*shape):
            return torch.nn.Parameter((torch.randn(*shape, generator=g) * init_std).to(dt).cuda())

        self.gate_w, self.w_up, self.w_down = p(E, H), p(E, I, H), p(E, H, I)
        self.w_gate = p(E, I, H) if cfg.hidden_act == api.ACT_SWIGLU else None

    def route(self, x):
        """The library's routing decision for x (no gradient): top-k indices and the packed-row tables."""
        with torch.no_grad():
            idx, _ = self.layer.gate(x.detach(), self.gate_w.detach())
            return idx, self.layer.route(idx)

    def gate_weights(self, x, idx):
        """The weights of the chosen experts, differentiable, by the formula the router kernel uses."""
        c = self.cfg
        logits = x.float() @ self.gate_w.float().t()
        scores = torch.softmax(logits, dim=1) if c.gate_fn == api.GATE_SOFTMAX else torch.sigmoid(logits)
        w = scores.gather(1, idx.long())
        return w / w.sum(1, keepdim=True) if c.norm_topk_prob else w

    def forward(self, x):
        c = self.cfg
        idx, r = self.route(x)
        count, offset = r["expert_count"], r["expert_offset"]
        tok = r["token_indices"].clamp(min=0).long()      # rows past the last kept one gather token 0 and are never used
        x_rows = x.index_select(0, tok)
        up = expert_linear(x_rows, self.w_up, self.layer, count, offset)
        gate = expert_linear(x_rows, self.w_gate, self.layer, count, offset) if c.hidden_act == api.ACT_SWIGLU else None
        y = act_down(up, gate, self.w_down, self.layer, count, offset)
        w = self.gate_weights(x, idx)
        rows = r["pair_row"]
        kept = (rows >= 0).unsqueeze(-1)
        picked = y.index_select(0, rows.clamp(min=0).reshape(-1).long()).reshape(c.tokens, c.expert_top_k, -1)
        out = (torch.where(kept, picked.float(), torch.zeros((), device=x.device)) * w.unsqueeze(-1)).sum(1)
        return out.to(x.dtype)
