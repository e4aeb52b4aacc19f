"""GPU behaviour at the edges of the contract: non-finite token rows, out-of-range expert ids from a caller, and a
dependency wait of the task queue that gives up (forced from the host, every kernel still exits normally)."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, to_device, upload_inputs

pytestmark = pytest.mark.gpu
FFN_TILED, FFN_PERSISTENT = 1, 2
STALL = 7   # MOE_ERR_QUEUE_STALL


@pytest.fixture(scope="module")
def moe():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import cuplayground_amd
    cuplayground_amd.load_library()
    return cuplayground_amd


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
@pytest.mark.parametrize("gate_fn", [ob.GATE_SOFTMAX, ob.GATE_SIGMOID], ids=["softmax", "sigmoid"])
def test_nan_token_row_keeps_routing_valid(moe, mode, gate_fn):
    """One NaN (or an overflow to inf - inf) in a token row makes all of that token's logits NaN.  The selection stays
    total (NaN ranks as -inf: experts 0..k-1), routing tables stay in range and bit-exact with the oracle, that
    token's output is NaN and every other token's output is what it is without the bad row."""
    import torch
    cfg = ob.Cfg(S=300, H=128, I=192, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, gate_fn=gate_fn, drop=0)
    inp = ob.make_inputs(cfg, seed=5)
    bad = [0, 17, 299]
    x = inp["x"].copy()
    x[17, 5] = 0x7FC0                       # bf16 NaN
    x[0, 3], x[0, 4] = 0x7F80, 0xFF80       # +inf and -inf: inf - inf in the dot product
    x[299, 127] = 0xFFC1
    inp_bad = dict(inp, x=x)
    want = ob.forward(cfg, inp_bad)
    for t in (17, 299):                     # every logit of these tokens is NaN
        assert list(want["topk_idx"][t]) == [0, 1]
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode)
    dev = upload_inputs(cfg, inp_bad)
    routing = layer.new_routing()
    out = layer.forward(dev["x"], dev, routing=routing)
    torch.cuda.synchronize()
    layer.task_counts()
    got = {k: from_device(v) for k, v in routing.items()}
    for key in ("topk_idx", "slot", "expert_count", "expert_offset", "token_indices"):
        assert np.array_equal(got[key], want[key]), key
    assert got["topk_idx"].min() >= 0 and got["topk_idx"].max() < cfg.E
    o = ob.to_f32(from_device(out), ob.BF16)
    ref = ob.to_f32(want["out"], ob.BF16)
    good = np.ones(cfg.S, bool)
    good[bad] = False
    assert np.isnan(o[[17, 299]]).all() and np.isnan(ref[[17, 299]]).all()
    assert np.array_equal(np.isnan(o[bad]), np.isnan(ref[bad]))   # the inf - inf token: NaN exactly where the oracle has it
    assert np.isfinite(o[good]).all()
    assert max_rel_err(o[good], ref[good]) <= OUT_TOL[ob.BF16]
    layer.close()


def test_route_drops_out_of_range_expert_ids(moe):
    """moe_route takes a caller's topk_idx: ids outside [0, E) are dropped instead of indexing past the tables."""
    import torch
    cfg = ob.Cfg(S=600, H=64, I=64, E=12, k=3, act=ob.ACT_RELU, dtype=ob.BF16, drop=1, capacity_factor=1.5)
    rng = np.random.default_rng(3)
    idx = rng.integers(0, cfg.E, size=(cfg.S, cfg.k)).astype(np.int32)
    hit = rng.random(idx.shape) < 0.05
    idx[hit] = rng.choice(np.array([-1, -2**31, cfg.E, 512, 2**31 - 1, 10**6], np.int64), size=hit.sum()).astype(np.int32)
    want = ob.route_slots(idx, cfg.E, cfg.drop, cfg.capacity)
    layer = moe.MoELayer(product_config(cfg))
    got = layer.route(to_device(idx, "i32"))
    torch.cuda.synchronize()
    for key in ("slot", "expert_count", "expert_offset", "token_indices", "pair_row"):
        assert np.array_equal(from_device(got[key]), want[key]), key
    assert (from_device(got["slot"])[hit] == -1).all()
    layer.close()


@pytest.mark.parametrize("name,cfg", [
    ("bf16", ob.Cfg(S=700, H=256, I=384, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0)),
    ("f32", ob.Cfg(S=200, H=128, I=128, E=4, k=1, act=ob.ACT_GELU, dtype=ob.F32, norm_topk=0, drop=0)),
    ("fp8", ob.Cfg(S=64, H=256, I=256, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0)),
    # enough rows per expert for the e4m3 tile GEMM instead of the weight streamer
    ("fp8_tile", ob.Cfg(S=600, H=256, I=256, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0)),
    # the fp32 matrix-core tile (forced: the layer is too small for the plan to pick it)
    ("f32_tile", ob.Cfg(S=600, H=256, I=128, E=2, k=1, act=ob.ACT_SWIGLU, dtype=ob.F32, norm_topk=0, drop=0)),
])
@pytest.mark.parametrize("combine", [0, 1, 2], ids=["combine_launch", "combine_arrivals", "combine_queue"])
def test_expired_dependency_wait_poisons_the_output_and_is_reported(moe, name, cfg, combine):
    """The queue kernel's bounded wait is made to give up from the host (spin limit < 0: every wait expires without
    polling).  Every kernel exits normally; no down-projection tile computes on unfinished rows -- its output is NaN,
    so every routed token's output is NaN; the stall is reported by the next calls on the handle without a
    synchronisation of their own, until it is cleared; after that the handle computes correctly again."""
    import torch
    inp = ob.make_inputs(cfg, seed=9)
    want = ob.forward(cfg, inp)
    # the combine inside the FFN kernels must carry the NaNs too
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT,
                         options={"combine": combine, "f32_tile": 1 if name == "f32_tile" else 0})
    assert name != "f32_tile" or layer.plan["block_rows"] == 128
    dev = upload_inputs(cfg, inp)
    layer.set_spin_limit(-1)
    out = layer.forward(dev["x"], dev)          # enqueues; the stall is not known yet
    torch.cuda.synchronize()
    o = ob.to_f32(from_device(out), cfg.act_dtype)
    routed = (want["slot"] >= 0).any(axis=1)
    assert routed.any() and np.isnan(o[routed]).all()
    with pytest.raises(moe.MoEError) as e:
        layer.forward(dev["x"], dev)
    assert e.value.status == STALL
    with pytest.raises(moe.MoEError) as e:
        layer.task_counts()
    assert e.value.status == STALL
    layer.clear_stall()
    layer.set_spin_limit(0)                      # back to the default
    out = layer.forward(dev["x"], dev)
    torch.cuda.synchronize()
    layer.task_counts()
    err = max_rel_err(ob.to_f32(from_device(out), cfg.act_dtype), ob.to_f32(want["out"], cfg.act_dtype))
    assert err <= OUT_TOL[cfg.dtype], err
    layer.close()


@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16], ids=["f32", "bf16"])
@pytest.mark.parametrize("act", [ob.ACT_RELU, ob.ACT_GELU, ob.ACT_NONE], ids=["relu", "gelu", "none"])
@pytest.mark.parametrize("M,N,K", [(40, 64, 64), (1100, 1024, 128)], ids=["small_tile", "large_tile"])
def test_gemm_epilogue_propagates_nan(moe, dtype, act, M, N, K):
    """A NaN accumulator stays a NaN through bias + activation (ReLU included, as with the reference's __hfma_relu,
    processor/tiling.cuh:45,54): a max-based ReLU would turn it into 0, a max-based identity into -inf."""
    rng = np.random.default_rng(1)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    A[3, 7] = np.nan
    A[M - 1, 0], A[M - 1, 1] = np.inf, -np.inf
    B[:, 0] = np.abs(B[:, 0]); B[:, 1] = np.abs(B[:, 1])      # inf * w0 - inf * w1: NaN in every column
    kind = "f32"
    if dtype == ob.BF16:
        A, B, kind = ob.f32_to_bf16(A), ob.f32_to_bf16(B), "bf16"
    got = ob.to_f32(from_device(moe.gemm_bias_act(to_device(A, kind), to_device(B, kind), None, act)), dtype)
    want = ob.to_f32(ob.gemm_bias_act(A, B, None, dtype, act), dtype)
    assert np.isnan(want[3]).all() and np.isnan(want[M - 1]).all()
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.abs(got[ok] - want[ok]).max() <= (1e-5 if dtype == ob.F32 else 1e-2) * np.abs(want[ok]).max()
