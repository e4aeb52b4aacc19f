"""The step before the path: bringing a model's expert weights into the layout `moe_forward` reads.

`moe_forward` takes, per layer, `gate_w [E,H]`, `w_up [E,I,H]`, `w_gate [E,I,H]` (SwiGLU), `w_down [E,H,I]` -- every
matrix (N,K) row-major with K innermost, the operand convention of the reference GEMM (`mma.cuh:417-419`) -- in the
activation dtype, or as e4m3 codes with one fp32 scale per 128 x 128 block (`torch_dtype` 4).  Checkpoints store one
small matrix per expert and projection instead.  This module

* packs such per-expert matrices into the stacked tensors (`pack_experts`), with the name mapping of Mixtral-style
  checkpoints built in (`pack_mixtral_block`: `experts.{e}.w1` is the SiLU-gated projection = `w_gate`, `w3` = `w_up`,
  `w2` = `w_down`, `gate.weight` = the router);
* quantises a packed set to the block-scaled e4m3 form on the GPU (`quantize_packed`, through `moe_quant_block128`);
* writes and reads a packed set as one safetensors file whose metadata carries the layer's knob file (`save_packed`,
  `load_packed`), so that a serving process maps the file and calls `moe_forward` without touching the weights again.

Nothing here computes on the CPU: packing is `torch.stack` on whatever device the tensors live on, quantisation runs
in the library.
"""
from __future__ import annotations

from typing import Dict, Mapping, Optional, Sequence

import torch

from . import api

PACKED_KEYS = ("gate_w", "gate_bias", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "s_up", "s_gate", "s_down",
               "prepared")


def pack_experts(gate_w: torch.Tensor, up: Sequence[torch.Tensor], down: Sequence[torch.Tensor],
                 gate_proj: Optional[Sequence[torch.Tensor]] = None, dtype: torch.dtype = torch.bfloat16,
                 device="cuda") -> Dict[str, torch.Tensor]:
    """Stacks per-expert matrices: `up[e]` and `gate_proj[e]` are [I,H], `down[e]` is [H,I] (torch.nn.Linear layout,
    which is already (N,K) row-major), `gate_w` is the router's [E,H]."""
    E = len(up)
    if len(down) != E or (gate_proj is not None and len(gate_proj) != E):
        raise ValueError("one up, one down (and one gate) projection per expert")
    I, H = up[0].shape
    for e in range(E):
        if tuple(up[e].shape) != (I, H) or tuple(down[e].shape) != (H, I):
            raise ValueError(f"expert {e}: expected up [{I},{H}] and down [{H},{I}]")
        if gate_proj is not None and tuple(gate_proj[e].shape) != (I, H):
            raise ValueError(f"expert {e}: expected gate projection [{I},{H}]")
    if tuple(gate_w.shape) != (E, H):
        raise ValueError(f"router weights must be [{E},{H}]")

    def stack(ms):
        return torch.stack([m.to(device=device, dtype=dtype) for m in ms]).contiguous()

    out = {"gate_w": gate_w.to(device=device, dtype=dtype).contiguous(), "w_up": stack(up), "w_down": stack(down)}
    if gate_proj is not None:
        out["w_gate"] = stack(gate_proj)
    return out


def pack_mixtral_block(state_dict: Mapping[str, torch.Tensor], prefix: str, dtype: torch.dtype = torch.bfloat16,
                       device="cuda") -> Dict[str, torch.Tensor]:
    """Packs one `block_sparse_moe` of a Mixtral-style checkpoint.  `prefix` is the block's key prefix, e.g.
    `model.layers.0.block_sparse_moe.`; the block computes `w2(silu(w1 x) * w3 x)` per expert."""
    gate_w = state_dict[prefix + "gate.weight"]
    E = gate_w.shape[0]
    name = prefix + "experts.{}.{}.weight"
    return pack_experts(gate_w, [state_dict[name.format(e, "w3")] for e in range(E)],
                        [state_dict[name.format(e, "w2")] for e in range(E)],
                        [state_dict[name.format(e, "w1")] for e in range(E)], dtype=dtype, device=device)


def mixtral_config(packed: Mapping[str, torch.Tensor], tokens: int, top_k: int = 2) -> api.MoEConfig:
    """The knob file of a Mixtral-style block for `tokens` rows per call: softmax router, top-k renormalised,
    SwiGLU, no token dropping."""
    E, I, H = packed["w_up"].shape
    fp8 = packed["w_up"].dtype in (torch.uint8, torch.float8_e4m3fn)
    return api.MoEConfig(capacity_factor=1.0, drop_tokens=0, expert_top_k=top_k, hidden_act=api.ACT_SWIGLU,
                         hidden_size=H, intermediate_size=I, micro_batch=1, num_experts=E, sequence_len=tokens,
                         torch_dtype=api.DTYPE_FP8 if fp8 else api.DTYPE_BF16, gate_fn=api.GATE_SOFTMAX,
                         norm_topk_prob=1)


def quantize_packed(packed: Mapping[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """bf16/fp32 expert matrices -> e4m3 codes + one fp32 scale per 128 x 128 block (scale = amax / 448); the router
    and the biases keep their dtype.  Runs on the GPU through `moe_quant_block128`."""
    out = {k: v for k, v in packed.items() if not k.startswith("w_")}
    for k in ("w_up", "w_gate", "w_down"):
        if k in packed:
            q, s = api.quantize_block128(packed[k])
            out[k] = q
            out["s_" + k[2:]] = s
    return out


def prepare_packed(packed: Mapping[str, torch.Tensor], layer: "api.MoELayer") -> Dict[str, torch.Tensor]:
    """Adds the kernel-ready operands of `layer`'s plan (`moe_prepare_weights`) to a packed set under the key
    "prepared" -- today the bf16 copies an e4m3 layer with many rows per expert would otherwise make in every call.
    They belong to the plan of `layer` (shape, dtype and options); a packed set saved with them serves handles of the
    same plan.  Returns `packed` unchanged when the plan prepares nothing."""
    out = dict(packed)
    out.pop("prepared", None)
    prepared = layer.prepare_weights(out)
    if prepared is not None:
        out["prepared"] = prepared
    return out


def save_packed(path: str, packed: Mapping[str, torch.Tensor], cfg: api.MoEConfig) -> None:
    """One safetensors file: the tensors under the argument names of `moe_forward` (the prepared operands included when
    the set carries them), the knob file in the metadata."""
    from safetensors.torch import save_file
    unknown = set(packed) - set(PACKED_KEYS)
    if unknown:
        raise ValueError(f"unknown tensors {sorted(unknown)}")
    save_file({k: v.contiguous().cpu() for k, v in packed.items()}, path,
              metadata={"moe355_config": cfg.to_json(), "moe355_format": "1"})


def load_packed(path: str, device="cuda"):
    """-> (tensors on `device`, MoEConfig).  The knob file is validated by the library's own loader."""
    from safetensors import safe_open
    tensors = {}
    with safe_open(path, framework="pt", device=str(device)) as f:
        meta = f.metadata() or {}
        if meta.get("moe355_format") != "1" or "moe355_config" not in meta:
            raise ValueError(f"{path} is not a packed moe355 layer")
        for k in f.keys():
            tensors[k] = f.get_tensor(k)
    return tensors, api.MoEConfig.from_json(meta["moe355_config"])


__all__ = ["pack_experts", "pack_mixtral_block", "mixtral_config", "quantize_packed", "prepare_packed", "save_packed", "load_packed",
           "PACKED_KEYS"]
