"""Shared test plumbing: oracle config <-> product config, numpy <-> device tensors, error metrics."""
import numpy as np

from oracle import binding as ob


def product_config(cfg: ob.Cfg):
    from cuplayground_amd import MoEConfig
    return MoEConfig(capacity_factor=cfg.capacity_factor, drop_tokens=cfg.drop, expert_top_k=cfg.k, hidden_act=cfg.act,
                     hidden_size=cfg.H, intermediate_size=cfg.I, micro_batch=1, num_experts=cfg.E,
                     sequence_len=cfg.S, torch_dtype=cfg.dtype, gate_fn=cfg.gate_fn, norm_topk_prob=cfg.norm_topk)


def to_device(a, kind):
    """kind: 'f32' | 'bf16' | 'f16' (numpy uint16 bit patterns) | 'u8' | 'i32'."""
    import torch
    if a is None:
        return None
    if kind in ("bf16", "f16"):
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).cuda().view(
            torch.bfloat16 if kind == "bf16" else torch.float16)
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def upload_inputs(cfg: ob.Cfg, inp: dict) -> dict:
    act = {ob.F32: "f32", ob.BF16: "bf16", ob.F16: "f16"}[cfg.act_dtype]
    wk = {ob.F32: "f32", ob.TF32: "f32", ob.BF16: "bf16", ob.F16: "f16", ob.FP8: "u8"}[cfg.dtype]
    kinds = dict(x=act, gate_w=act, gate_bias="f32", w_up=wk, w_gate=wk, w_down=wk, b_up=act, b_gate=act, b_down=act,
                 s_up="f32", s_gate="f32", s_down="f32")
    return {n: to_device(inp.get(n), kinds[n]) for n in kinds if inp.get(n) is not None}


def from_device(t):
    """device tensor -> numpy; bf16 and fp16 come back as uint16 bit patterns."""
    import torch
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).cpu().numpy().view(np.uint16)
    return t.cpu().numpy()


def as_f32(a, dtype):
    return ob.to_f32(a, ob.Cfg(S=1, H=1, I=1, E=1, k=1, dtype=dtype).act_dtype)


def max_rel_err(y, ref):
    """max|y - ref| / max|ref| -- the metric the output tolerance is stated in."""
    y = np.asarray(y, np.float64); ref = np.asarray(ref, np.float64)
    return float(np.abs(y - ref).max() / max(np.abs(ref).max(), 1e-30))


# fp16 carries 11 significant bits against bf16's 8: its bound is an eighth of bf16's
OUT_TOL = {ob.F32: 1e-5, ob.TF32: 1e-5, ob.BF16: 1e-2, ob.F16: 1.25e-3, ob.FP8: 3e-2}
