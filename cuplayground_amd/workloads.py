"""The five layer shapes the operator is measured and tested on, as `MoEConfig`s, and their synthetic operands.

Shapes (tokens S = micro_batch x sequence_len; knob names are those of aristos_config.json,
aristos_config.schema.json:5-58):
  tiny         S=128   H=256  I=512   E=8   top-1 softmax, capacity factor 1.0,  GELU,   fp32
  mid          S=4096  H=2048 I=2048  E=16  top-2 softmax renormalised, cf 1.25, GELU,   bf16
  mixtral      S=8192  H=4096 I=14336 E=8   top-2, SwiGLU, bf16, no token dropping
  finegrained  S=16384 H=2048 I=1408  E=64  top-6, SwiGLU, bf16, cf 1.0, per-expert logit bias ~ Zipf(1.1) loads
  decode_fp8   S=64    H=7168 I=2048  E=256 top-8 sigmoid, SwiGLU, e4m3 weights with 128x128 block scales, bf16 tokens
Tokens are N(0,1), gate and expert weights N(0,0.02), rounded once to their storage types.
Two more shapes, not among the five:
  prefill_fp8        the mixtral shape with e4m3 weights and 128x128 block scales (bf16 tokens, bf16 MFMA arithmetic)
  reference_default  the reference's own aristos_config.json: S=8192 H=1024 I=4096 E=1 top-1, ReLU, fp32
"""
from __future__ import annotations

from dataclasses import dataclass

from . import api


@dataclass(frozen=True)
class Workload:
    tag: str                 # C1..C5
    config: api.MoEConfig
    zipf_bias: bool = False  # per-expert gate bias log(p_e), p_e ~ rank^-1.1
    bound: str = "mfma"      # the roofline the FFN stage is held against

    def describe(self) -> str:
        c = self.config
        act = {api.ACT_RELU: "relu", api.ACT_GELU: "gelu", api.ACT_SWIGLU: "swiglu"}[c.hidden_act]
        drop = "drop cf=%g" % c.capacity_factor if c.drop_tokens else "dropless"
        return "%s: S=%d H=%d I=%d E=%d top%d %s %s" % (self.tag, c.tokens, c.hidden_size, c.intermediate_size,
                                                        c.num_experts, c.expert_top_k, act, drop)


def _cfg(S, H, I, E, k, act, dtype, cf, drop, gate_fn=api.GATE_SOFTMAX, norm=1):
    return api.MoEConfig(capacity_factor=cf, drop_tokens=drop, expert_top_k=k, hidden_act=act, hidden_size=H,
                         intermediate_size=I, micro_batch=1, num_experts=E, sequence_len=S, torch_dtype=dtype,
                         gate_fn=gate_fn, norm_topk_prob=norm)


WORKLOADS = {
    "tiny": Workload("C1", _cfg(128, 256, 512, 8, 1, api.ACT_GELU, api.DTYPE_F32, 1.0, 1, norm=0), bound="hbm"),
    "mid": Workload("C2", _cfg(4096, 2048, 2048, 16, 2, api.ACT_GELU, api.DTYPE_BF16, 1.25, 1)),
    "mixtral": Workload("C3", _cfg(8192, 4096, 14336, 8, 2, api.ACT_SWIGLU, api.DTYPE_BF16, 2.0, 0)),
    "finegrained": Workload("C4", _cfg(16384, 2048, 1408, 64, 6, api.ACT_SWIGLU, api.DTYPE_BF16, 1.0, 1),
                            zipf_bias=True),
    "decode_fp8": Workload("C5", _cfg(64, 7168, 2048, 256, 8, api.ACT_SWIGLU, api.DTYPE_FP8, 1.0, 0,
                                      gate_fn=api.GATE_SIGMOID), bound="hbm"),
    "prefill_fp8": Workload("X1", _cfg(8192, 4096, 14336, 8, 2, api.ACT_SWIGLU, api.DTYPE_FP8, 2.0, 0)),
    # the knob file the reference ships (aristos_config.json): one expert, fp32, ReLU, 4 x 2048 tokens
    "reference_default": Workload("R0", _cfg(8192, 1024, 4096, 1, 1, api.ACT_RELU, api.DTYPE_F32, 1.0, 0, norm=0)),
}


def zipf_gate_bias(E: int, seed: int, s: float = 1.1):
    """log(p_e) with p_e proportional to rank_e^-s under a seeded random ranking of the experts (numpy fp32 [E])."""
    import numpy as np
    rank = np.random.default_rng(seed).permutation(E).astype(np.float64) + 1.0
    p = rank ** (-s)
    return np.log(p / p.sum()).astype(np.float32)


def make_device_inputs(w: Workload, seed: int = 42) -> dict:
    """Synthetic operands generated on the current GPU under the argument names of moe_forward."""
    import torch
    c = w.config
    g = torch.Generator(device="cuda").manual_seed(seed)
    adt = torch.float32 if c.torch_dtype == api.DTYPE_F32 else torch.bfloat16
    S, H, I, E = c.tokens, c.hidden_size, c.intermediate_size, c.num_experts

    def normal(shape, std, dtype):
        out = torch.empty(shape, dtype=dtype, device="cuda")
        for i in range(shape[0]):      # expert by expert: bounds the fp32 temporary
            out[i] = (torch.randn(shape[1:], generator=g, device="cuda", dtype=torch.float32) * std).to(dtype)
        return out

    d = {"x": torch.randn(S, H, generator=g, device="cuda", dtype=torch.float32).to(adt),
         "gate_w": (torch.randn(E, H, generator=g, device="cuda", dtype=torch.float32) * 0.02).to(adt)}
    if w.zipf_bias:
        d["gate_bias"] = torch.from_numpy(zipf_gate_bias(E, seed)).cuda()
    names = ["w_up", "w_down"] + (["w_gate"] if c.hidden_act == api.ACT_SWIGLU else [])
    for n in names:
        shape = (E, H, I) if n == "w_down" else (E, I, H)
        if c.torch_dtype == api.DTYPE_FP8:
            wf = normal(shape, 0.02, torch.float32)
            d[n], d["s_" + n[2:]] = api.quantize_block128(wf)   # e4m3 codes + one scale per 128x128 block
            del wf
        else:
            d[n] = normal(shape, 0.02, adt)
    return d


def balance_routing(c: api.MoEConfig, dev: dict) -> None:
    """Rewrites the router's inputs in place so that token t picks experts t, t+1, .. t+k-1 (mod E): every expert
    receives exactly S*k/E rows.  Only the first E columns of x and the gate weights change (E of H columns), so the
    FFN does the same arithmetic on (almost) the same data; used to measure what ragged last row blocks cost."""
    import torch
    E, k = c.num_experts, c.expert_top_k
    x, gw = dev["x"], dev["gate_w"]
    gw.zero_()
    x[:, :E] = 0
    t = torch.arange(c.tokens, device=x.device)
    for r in range(k):
        x[t, (t + r) % E] = 40.0
    gw[:, :E] = torch.eye(E, device=x.device, dtype=gw.dtype)
    if dev.get("gate_bias") is not None:
        dev["gate_bias"].zero_()


def ffn_flops(c: api.MoEConfig, kept_rows: int) -> float:
    """2 * g * H * I per kept (token, expert) row; g = 3 matrices for SwiGLU, 2 otherwise."""
    g = 3 if c.hidden_act == api.ACT_SWIGLU else 2
    return 2.0 * g * kept_rows * c.hidden_size * c.intermediate_size


def fp8_ffn_bytes(c: api.MoEConfig, active_experts: int, kept_rows: int) -> float:
    """Bytes the decode-shaped FFN has to move once: the e4m3 weights and block scales of every expert that received
    a row, the gathered token rows in and the expert output rows out (bf16)."""
    H, I = c.hidden_size, c.intermediate_size
    scale_bytes = 3 * (H // 128) * (I // 128) * 4
    return active_experts * (3.0 * H * I + scale_bytes) + 2.0 * kept_rows * H * 2
