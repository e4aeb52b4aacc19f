"""Packing of per-expert checkpoint matrices into the operand layout of moe_forward (host logic; runs on the CPU)."""
import pytest
import torch

from cuplayground_amd import api
from cuplayground_amd import weights as W


def mixtral_like_state_dict(E=4, H=64, I=128, seed=0, prefix="model.layers.3.block_sparse_moe."):
    g = torch.Generator().manual_seed(seed)
    sd = {prefix + "gate.weight": torch.randn(E, H, generator=g)}
    for e in range(E):
        sd[prefix + f"experts.{e}.w1.weight"] = torch.randn(I, H, generator=g)
        sd[prefix + f"experts.{e}.w2.weight"] = torch.randn(H, I, generator=g)
        sd[prefix + f"experts.{e}.w3.weight"] = torch.randn(I, H, generator=g)
    return sd, prefix


def test_mixtral_names_map_to_the_operands():
    sd, prefix = mixtral_like_state_dict()
    p = W.pack_mixtral_block(sd, prefix, dtype=torch.bfloat16, device="cpu")
    assert set(p) == {"gate_w", "w_up", "w_gate", "w_down"}
    assert p["w_up"].shape == (4, 128, 64) and p["w_gate"].shape == (4, 128, 64) and p["w_down"].shape == (4, 64, 128)
    assert all(t.is_contiguous() and t.dtype == torch.bfloat16 for t in p.values())
    for e in range(4):      # w1 carries the SiLU: it is the gate projection; w3 is the up projection
        assert torch.equal(p["w_gate"][e], sd[prefix + f"experts.{e}.w1.weight"].bfloat16())
        assert torch.equal(p["w_up"][e], sd[prefix + f"experts.{e}.w3.weight"].bfloat16())
        assert torch.equal(p["w_down"][e], sd[prefix + f"experts.{e}.w2.weight"].bfloat16())
    assert torch.equal(p["gate_w"], sd[prefix + "gate.weight"].bfloat16())
    cfg = W.mixtral_config(p, tokens=256)
    assert (cfg.num_experts, cfg.hidden_size, cfg.intermediate_size, cfg.expert_top_k) == (4, 64, 128, 2)
    assert cfg.hidden_act == api.ACT_SWIGLU and cfg.norm_topk_prob == 1 and cfg.drop_tokens == 0
    assert cfg.torch_dtype == api.DTYPE_BF16 and cfg.tokens == 256
    cfg.validate()


def test_shape_errors():
    sd, prefix = mixtral_like_state_dict()
    up = [sd[prefix + f"experts.{e}.w3.weight"] for e in range(4)]
    down = [sd[prefix + f"experts.{e}.w2.weight"] for e in range(4)]
    with pytest.raises(ValueError):
        W.pack_experts(sd[prefix + "gate.weight"], up, down[:3], device="cpu")
    with pytest.raises(ValueError):
        W.pack_experts(sd[prefix + "gate.weight"], up, [d.t() for d in down], device="cpu")
    with pytest.raises(ValueError):
        W.pack_experts(sd[prefix + "gate.weight"][:3], up, down, device="cpu")


def test_file_round_trip(tmp_path):
    sd, prefix = mixtral_like_state_dict(seed=1)
    p = W.pack_mixtral_block(sd, prefix, device="cpu")
    p["s_up"] = torch.rand(4, 1, 1)                       # any of the operand names may be stored
    cfg = W.mixtral_config(p, tokens=128)
    path = str(tmp_path / "layer.safetensors")
    W.save_packed(path, p, cfg)
    q, cfg2 = W.load_packed(path, device="cpu")
    assert cfg2 == cfg
    assert set(q) == set(p) and all(torch.equal(q[k], p[k]) for k in p)
    with pytest.raises(ValueError):
        W.save_packed(path, {"weights": p["w_up"]}, cfg)
    from safetensors.torch import save_file
    other = str(tmp_path / "other.safetensors")
    save_file({"w_up": p["w_up"]}, other)
    with pytest.raises(ValueError):
        W.load_packed(other, device="cpu")
