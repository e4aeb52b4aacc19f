"""Pins the oracle's whole-layer function by the dense-mixture equivalence in float64."""
import numpy as np
import pytest
from scipy.special import erf

from oracle import binding as ob


def dense_mixture(cfg, inp, routing):
    """out[t] = sum_r w[t,r] * FFN_{e(t,r)}(x[t]) for every kept pair, all in float64, token by token."""
    adt = cfg.act_dtype
    x = ob.to_f32(inp["x"], adt).astype(np.float64)

    def weight(name):
        if cfg.dtype == ob.FP8:
            return ob.dequant_block128(inp[name], inp["s_" + name[2:]]).astype(np.float64)
        return ob.to_f32(inp[name], cfg.dtype).astype(np.float64)

    wu, wd = weight("w_up"), weight("w_down")
    wg = weight("w_gate") if cfg.act == ob.ACT_SWIGLU else None
    bias = {n: ob.to_f32(inp[n], adt).astype(np.float64) if inp.get(n) is not None else None
            for n in ("b_up", "b_gate", "b_down")}
    out = np.zeros((cfg.S, cfg.H))
    for t in range(cfg.S):
        for r in range(cfg.k):
            if routing["slot"][t, r] < 0:
                continue
            e = routing["topk_idx"][t, r]
            u = wu[e] @ x[t] + (bias["b_up"][e] if bias["b_up"] is not None else 0)
            if cfg.act == ob.ACT_SWIGLU:
                g = wg[e] @ x[t] + (bias["b_gate"][e] if bias["b_gate"] is not None else 0)
                h = g / (1 + np.exp(-g)) * u
            elif cfg.act == ob.ACT_GELU:
                h = 0.5 * u * (1 + erf(u / np.sqrt(2)))
            else:
                h = np.maximum(u, 0)
            y = wd[e] @ h + (bias["b_down"][e] if bias["b_down"] is not None else 0)
            out[t] += np.float64(routing["topk_w"][t, r]) * y
    return out


CASES = {
    "f32_gelu_top1_drop": ob.Cfg(S=96, H=128, I=192, E=6, k=1, act=ob.ACT_GELU, dtype=ob.F32, norm_topk=0, drop=1,
                                 capacity_factor=1.0),
    "f32_relu_top2": ob.Cfg(S=64, H=64, I=128, E=4, k=2, act=ob.ACT_RELU, dtype=ob.F32, norm_topk=1, drop=0),
    "f32_swiglu_top3_bias": ob.Cfg(S=48, H=128, I=64, E=8, k=3, act=ob.ACT_SWIGLU, dtype=ob.F32, norm_topk=1, drop=1,
                                   capacity_factor=0.5),
    "bf16_gelu_top2": ob.Cfg(S=80, H=128, I=256, E=5, k=2, act=ob.ACT_GELU, dtype=ob.BF16, norm_topk=1, drop=1,
                             capacity_factor=1.25),
    "bf16_swiglu_sigmoid": ob.Cfg(S=40, H=192, I=128, E=16, k=4, act=ob.ACT_SWIGLU, dtype=ob.BF16,
                                  gate_fn=ob.GATE_SIGMOID, norm_topk=1, drop=0),
    "fp16_swiglu_top2_bias": ob.Cfg(S=72, H=128, I=192, E=6, k=2, act=ob.ACT_SWIGLU, dtype=ob.F16, norm_topk=1, drop=1,
                                    capacity_factor=1.0),
    "fp16_gelu_top1": ob.Cfg(S=50, H=64, I=128, E=3, k=1, act=ob.ACT_GELU, dtype=ob.F16, norm_topk=0, drop=0),
    "tf32_relu_top2": ob.Cfg(S=40, H=64, I=64, E=4, k=2, act=ob.ACT_RELU, dtype=ob.TF32, norm_topk=1, drop=0),
    "fp8_swiglu_sigmoid": ob.Cfg(S=24, H=256, I=128, E=12, k=3, act=ob.ACT_SWIGLU, dtype=ob.FP8,
                                 gate_fn=ob.GATE_SIGMOID, norm_topk=1, drop=0),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_layer_equals_dense_mixture(name):
    cfg = CASES[name]
    inp = ob.make_inputs(cfg, seed=11, with_bias="bias" in name)
    r = ob.forward(cfg, inp)
    routing = ob.route(cfg, inp)
    for key in ("topk_idx", "slot", "expert_count", "expert_offset", "token_indices"):
        assert np.array_equal(r[key], routing[key]), key
    assert np.array_equal(r["topk_w"], routing["topk_w"])
    want = dense_mixture(cfg, inp, r)
    got = ob.to_f32(r["out"], cfg.act_dtype)
    # storage rounding of h, y and out (bf16: 2^-9 relative each) is the only difference from float64
    tol = {ob.F32: 1e-5, ob.TF32: 1e-5, ob.F16: 1.25e-3}.get(cfg.dtype, 1e-2)
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
    assert np.abs(want).max() > 0
    # dropped-everywhere tokens are exactly zero
    dead = (r["slot"] < 0).all(axis=1)
    assert (got[dead] == 0).all()
    if cfg.drop and cfg.capacity_factor < 1.0:
        assert dead.any() or (r["slot"] < 0).any()
    # the sampled path used at full size reproduces the full path row for row
    tokens = np.arange(0, cfg.S, 3, dtype=np.int32)
    rows = ob.forward_tokens(cfg, inp, r["topk_idx"], r["topk_w"], r["slot"], tokens)
    assert np.array_equal(rows, r["out"][tokens])


def test_ffn_rows_is_two_chained_reference_gemms():
    """One FFN row = the reference GEMM contract applied twice, intermediate rounded to storage in between."""
    cfg = ob.Cfg(S=8, H=64, I=128, E=2, k=1, act=ob.ACT_GELU, dtype=ob.BF16)
    inp = ob.make_inputs(cfg, seed=5, with_bias=True)
    tokens = np.arange(8, dtype=np.int32); experts = (tokens % 2).astype(np.int32)
    y = ob.ffn_rows(cfg, inp, tokens, experts)
    for e in range(2):
        sel = experts == e
        h = ob.gemm_bias_act(inp["x"][sel], inp["w_up"][e], inp["b_up"][e], ob.BF16, ob.ACT_GELU)
        want = ob.gemm_bias_act(h, inp["w_down"][e], inp["b_down"][e], ob.BF16, ob.ACT_NONE)
        assert np.array_equal(y[sel], want)


def test_zipf_bias_skews_expert_load():
    cfg = ob.BASELINE["C4"].scaled(S=2048)
    inp = ob.make_inputs(ob.Cfg(S=cfg.S, H=cfg.H, I=64, E=cfg.E, k=cfg.k, act=ob.ACT_SWIGLU, dtype=ob.BF16,
                                zipf_bias=True))
    b = inp["gate_bias"]
    assert np.isclose(np.exp(b.astype(np.float64)).sum(), 1.0, atol=1e-5)
    p = np.sort(np.exp(b.astype(np.float64)))[::-1]
    assert np.allclose(p / p[0], np.arange(1, cfg.E + 1) ** -1.1, rtol=1e-4)
    logits = ob.gate_logits(inp["x"], inp["gate_w"], b, ob.BF16)
    idx, _ = ob.topk(logits, cfg.k, ob.GATE_SOFTMAX, 1)
    load = np.bincount(idx.reshape(-1), minlength=cfg.E)
    assert load[np.argmax(b)] == load.max() and load.max() > 5 * np.median(load)
