"""`torch.ops.moe355.forward`: the MoE layer as a PyTorch operator over the C ABI of libmoe355.

The operator takes the knob file of the reference (`aristos_config.json`, schema `aristos_config.schema.json:5-71`)
as a JSON string plus the layer's tensors, and runs `moe_forward` on the current CUDA(HIP) stream.  Only a CUDA
implementation (and a meta implementation for shape inference) is registered: called with CPU tensors the dispatcher
raises, there is no CPU path.  `MoE355` wraps it as an `nn.Module`; `torch_reference` is the same layer written with
plain torch ops (fp32 accumulation, one rounding of the intermediate and of the output), for in-process comparison.
"""
from __future__ import annotations

import json

import torch

from . import api

_SCHEMA = ("forward(Tensor x, Tensor gate_w, Tensor w_up, Tensor? w_gate, Tensor w_down, str config, "
           "Tensor? gate_bias=None, Tensor? b_up=None, Tensor? b_gate=None, Tensor? b_down=None, "
           "Tensor? s_up=None, Tensor? s_gate=None, Tensor? s_down=None) -> Tensor")
_lib = torch.library.Library("moe355", "DEF")
_lib.define(_SCHEMA)

_layers: dict = {}   # (config text, device index) -> api.MoELayer (handle + workspace, reused across calls)


def _layer_for(config: str, device: torch.device) -> api.MoELayer:
    key = (config, device.index if device.index is not None else torch.cuda.current_device())
    layer = _layers.get(key)
    if layer is None:
        with torch.cuda.device(key[1]):
            layer = api.MoELayer(api.MoEConfig.from_json(config))
        _layers[key] = layer
    return layer


def _check_tensor(name, t, shape, dtypes):
    if t is None:
        return
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")
    if t.dtype not in dtypes:
        raise ValueError(f"{name}: expected dtype in {dtypes}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous (row-major, K innermost)")
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU")


def _forward_cuda(x, gate_w, w_up, w_gate, w_down, config, gate_bias=None, b_up=None, b_gate=None, b_down=None,
                  s_up=None, s_gate=None, s_down=None):
    layer = _layer_for(config, x.device)
    cfg = layer.cfg
    S, H, I, E = cfg.tokens, cfg.hidden_size, cfg.intermediate_size, cfg.num_experts
    act = layer.act_dtype
    fp8 = cfg.torch_dtype == api.DTYPE_FP8
    wdt = (torch.float8_e4m3fn, torch.uint8) if fp8 else (act,)
    _check_tensor("x", x, (S, H), (act,))
    _check_tensor("gate_w", gate_w, (E, H), (act,))
    _check_tensor("gate_bias", gate_bias, (E,), (torch.float32,))
    _check_tensor("w_up", w_up, (E, I, H), wdt)
    _check_tensor("w_gate", w_gate, (E, I, H), wdt)
    _check_tensor("w_down", w_down, (E, H, I), wdt)
    _check_tensor("b_up", b_up, (E, I), (act,))
    _check_tensor("b_gate", b_gate, (E, I), (act,))
    _check_tensor("b_down", b_down, (E, H), (act,))
    if cfg.hidden_act == api.ACT_SWIGLU and w_gate is None:
        raise ValueError("hidden_act = swiglu needs w_gate")
    if fp8:
        _check_tensor("s_up", s_up, (E, I // 128, H // 128), (torch.float32,))
        _check_tensor("s_gate", s_gate, (E, I // 128, H // 128), (torch.float32,))
        _check_tensor("s_down", s_down, (E, H // 128, I // 128), (torch.float32,))
        if s_up is None or s_down is None:
            raise ValueError("torch_dtype = fp8 needs the block scales s_up and s_down")
    weights = dict(gate_w=gate_w, gate_bias=gate_bias, w_up=w_up, w_gate=w_gate, w_down=w_down, b_up=b_up,
                   b_gate=b_gate, b_down=b_down, s_up=s_up, s_gate=s_gate, s_down=s_down)
    with torch.cuda.device(x.device):
        return layer.forward(x, weights)


def _forward_meta(x, gate_w, w_up, w_gate, w_down, config, gate_bias=None, b_up=None, b_gate=None, b_down=None,
                  s_up=None, s_gate=None, s_down=None):
    return torch.empty_like(x)


_lib.impl("forward", _forward_cuda, "CUDA")
_lib.impl("forward", _forward_meta, "Meta")


class MoE355(torch.nn.Module):
    """One MoE layer with its weights; forward(x[S,H]) -> [S,H] through torch.ops.moe355.forward.

    Built either with random weights (`MoE355(cfg)`, bf16/f32 only) or from packed tensors under the argument names of
    `moe_forward` (`MoE355.from_packed(cfg, tensors)`; see `cuplayground_amd.weights` for packing, quantising and
    loading them), which also covers the block-scaled e4m3 layers."""

    _NAMES = ("gate_w", "gate_bias", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "s_up", "s_gate", "s_down")

    def __init__(self, cfg: api.MoEConfig, device="cuda", init_std: float = 0.02, seed: int = 0, tensors=None):
        super().__init__()
        self.cfg = cfg
        self.config_json = cfg.to_json()
        if tensors is None:
            if cfg.torch_dtype == api.DTYPE_FP8:
                raise ValueError("build fp8 layers from quantised tensors: MoE355.from_packed(cfg, tensors)")
            dt = api._torch_act_dtype(cfg.torch_dtype)
            E, H, I = cfg.num_experts, cfg.hidden_size, cfg.intermediate_size
            g = torch.Generator(device="cpu").manual_seed(seed)

            def w(*shape):
                return (torch.randn(*shape, generator=g) * init_std).to(dt).to(device)

            tensors = {"gate_w": w(E, H), "w_up": w(E, I, H), "w_down": w(E, H, I)}
            if cfg.hidden_act == api.ACT_SWIGLU:
                tensors["w_gate"] = w(E, I, H)
        unknown = set(tensors) - set(self._NAMES)
        if unknown:
            raise ValueError(f"unknown tensors {sorted(unknown)}")
        for name in self._NAMES:       # buffers: inference weights, integer codes included
            t = tensors.get(name)
            self.register_buffer(name, None if t is None else t.to(device).contiguous())

    @classmethod
    def from_packed(cls, cfg: api.MoEConfig, tensors, device="cuda") -> "MoE355":
        return cls(cfg, device=device, tensors=tensors)

    def forward(self, x):
        return torch.ops.moe355.forward(x, self.gate_w, self.w_up, self.w_gate, self.w_down, self.config_json,
                                        self.gate_bias, self.b_up, self.b_gate, self.b_down, self.s_up, self.s_gate,
                                        self.s_down)

    def reference(self, x):
        return torch_reference(x, self.cfg, self.gate_w, self.w_up, self.w_gate, self.w_down, gate_bias=self.gate_bias)


def torch_reference(x, cfg: api.MoEConfig, gate_w, w_up, w_gate, w_down, gate_bias=None, topk=None):
    """The layer in plain torch ops, for comparison in the same process.

    fp32 accumulation everywhere, the intermediate and the output rounded once to the storage dtype; capacity drops by
    stable order of the flattened (token, rank) pairs.  The router's fp32 sum runs in torch's order, not in the order
    the kernels fix, so on near-ties the selected experts can differ; pass `topk=(idx, w)` to take the routing from
    elsewhere.
    """
    S, k, E = x.shape[0], cfg.expert_top_k, cfg.num_experts
    xf = x.float()
    if topk is None:
        logits = xf @ gate_w.float().t()
        if gate_bias is not None:
            logits = logits + gate_bias
        vals, idx = torch.topk(logits, k, dim=1)
        if cfg.gate_fn == api.GATE_SOFTMAX:
            w = torch.exp(vals - vals[:, :1]) / torch.exp(logits - vals[:, :1]).sum(1, keepdim=True)
        else:
            w = torch.sigmoid(vals)
        if cfg.norm_topk_prob:
            w = w / w.sum(1, keepdim=True)
    else:
        idx, w = topk[0].long(), topk[1].float()
    flat = idx.reshape(-1)
    order = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=E)
    starts = torch.cumsum(counts, 0) - counts
    slot = torch.empty_like(flat)
    slot[order] = torch.arange(flat.numel(), device=flat.device) - starts[flat[order]]
    keep = torch.ones_like(flat, dtype=torch.bool)
    if cfg.drop_tokens:
        keep = slot < cfg.capacity
    dt = x.dtype
    out = torch.zeros(S, x.shape[1], dtype=torch.float32, device=x.device)
    tok = torch.arange(S, device=x.device).repeat_interleave(k)
    for r in range(k):                      # ascending rank, as the combine stage sums
        sel = (torch.arange(flat.numel(), device=x.device) % k) == r
        for e in range(E):
            m = sel & keep & (flat == e)
            if not bool(m.any()):
                continue
            t = tok[m]
            xe = xf[t]
            up = xe @ w_up[e].float().t()
            if cfg.hidden_act == api.ACT_SWIGLU:
                h = torch.nn.functional.silu(xe @ w_gate[e].float().t()) * up
            elif cfg.hidden_act == api.ACT_GELU:
                h = torch.nn.functional.gelu(up)
            else:
                h = torch.relu(up)
            y = (h.to(dt).float() @ w_down[e].float().t()).to(dt).float()
            out[t] += w.reshape(-1)[m].unsqueeze(1) * y
    return out.to(dt)


def torch_cpu_layer(x, cfg: api.MoEConfig, gate_w, w_up, w_gate, w_down, gate_bias=None):
    """The layer as a libtorch program on the host -- the CPU computation the reference reserves a hook for and leaves
    empty (`torching.cuh:7-11`, libtorch linked at `CMakeLists.txt:126-133`): linear -> softmax / sigmoid -> topk ->
    stable sort by expert -> index_select -> per-expert linear / activation / linear -> index_add.  Tensors live on
    the CPU; matmuls run in the dtype of the weights handed in (hand fp32 weights for fp32 accumulation from bf16
    storage), the intermediate and the output are rounded to x.dtype.  Used as the timed CPU baseline; also runs on
    GPU tensors.  Returns (out [S,H], topk_idx [S,k])."""
    F = torch.nn.functional
    S, k, E = x.shape[0], cfg.expert_top_k, cfg.num_experts
    cdt = w_up.dtype
    logits = F.linear(x.float(), gate_w.float())
    if gate_bias is not None:
        logits = logits + gate_bias
    scores = torch.softmax(logits, dim=1) if cfg.gate_fn == api.GATE_SOFTMAX else torch.sigmoid(logits)
    w, idx = torch.topk(scores, k, dim=1)
    if cfg.norm_topk_prob:
        w = w / w.sum(1, keepdim=True)
    flat = idx.reshape(-1)
    order = torch.sort(flat, stable=True).indices           # pairs grouped by expert, token order kept
    counts = torch.bincount(flat, minlength=E)
    starts = torch.cumsum(counts, 0) - counts
    kept = torch.clamp(counts, max=cfg.capacity) if cfg.drop_tokens else counts
    out = torch.zeros(S, x.shape[1], dtype=torch.float32, device=x.device)
    wflat = w.reshape(-1)
    for e in range(E):
        n = int(kept[e])
        if n == 0:
            continue
        pairs = order[int(starts[e]):int(starts[e]) + n]
        tok = pairs // k
        xe = x.index_select(0, tok).to(cdt)
        up = F.linear(xe, w_up[e])
        if cfg.hidden_act == api.ACT_SWIGLU:
            h = F.silu(F.linear(xe, w_gate[e])) * up
        elif cfg.hidden_act == api.ACT_GELU:
            h = F.gelu(up)
        else:
            h = torch.relu(up)
        y = F.linear(h.to(x.dtype).to(cdt), w_down[e]).to(x.dtype).float()
        out.index_add_(0, tok, y * wflat[pairs].unsqueeze(1))
    return out.to(x.dtype), idx


__all__ = ["MoE355", "torch_reference", "torch_cpu_layer"]
