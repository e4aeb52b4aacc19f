"""GPU parity of the single stages, called through the C ABI, against the CPU oracle."""
import hashlib
import json
import os

import numpy as np
import pytest

from oracle import binding as ob
from helpers import from_device, product_config, to_device, upload_inputs
from test_oracle_gemm_combine import collective_operands

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def moe():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import cuplayground_amd
    cuplayground_amd.load_library()
    return cuplayground_amd


def bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


# ---------------------------------------------------------------- GEMM + epilogue (reference fGET contract)
KIND = {ob.F32: "f32", ob.BF16: "bf16", ob.F16: "f16"}


@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16, ob.F16])
def test_gemm_reference_driver_known_answer(moe, dtype):
    """testCollective's operands (mma.cuh:394-411): closed-form expected output."""
    A, B, bias, want = collective_operands(dtype)
    kind = KIND[dtype]
    C = moe.gemm_bias_act(to_device(A, kind), to_device(B, kind), to_device(bias, kind), ob.ACT_RELU)
    got = ob.to_f32(from_device(C), dtype)
    assert got[0, 0] == 6 and got[0, 1] == 9 and got[1, 0] == 24 and got[1, 1] == 35
    assert np.array_equal(got, want)


@pytest.mark.parametrize("act", [ob.ACT_RELU, ob.ACT_GELU, ob.ACT_NONE])
@pytest.mark.parametrize("dtype,M,N,K", [(ob.F32, 100, 66, 48), (ob.F32, 64, 128, 256),
                                         (ob.F32, 2100, 2048, 160),     # 17 x 16 tiles of 128 x 128: the matrix-core tile, ragged last block
                                         (ob.BF16, 300, 200, 192),
                                         (ob.BF16, 128, 128, 64), (ob.BF16, 1, 4, 64), (ob.BF16, 129, 260, 1024),
                                         (ob.F16, 300, 200, 192), (ob.F16, 129, 260, 1024), (ob.F16, 1100, 1024, 256)])
def test_gemm_vs_oracle(moe, dtype, M, N, K, act):
    rng = np.random.default_rng(M * 7 + N)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = (rng.standard_normal((N, K)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    kind = KIND[dtype]
    A, B, bias = ob.from_f32(A, dtype), ob.from_f32(B, dtype), ob.from_f32(bias, dtype)
    want = ob.to_f32(ob.gemm_bias_act(A, B, bias, dtype, act), dtype)
    got = ob.to_f32(from_device(moe.gemm_bias_act(to_device(A, kind), to_device(B, kind), to_device(bias, kind), act)),
                    dtype)
    tol = {ob.F32: 1e-5, ob.BF16: 1e-2, ob.F16: 1.25e-3}[dtype]   # fp32: summation order only; bf16 / fp16: an output ulp is 2^-8 / 2^-11
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
    got_nb = ob.to_f32(from_device(moe.gemm_bias_act(to_device(A, kind), to_device(B, kind), None, act)), dtype)
    want_nb = ob.to_f32(ob.gemm_bias_act(A, B, None, dtype, act), dtype)
    assert np.abs(got_nb - want_nb).max() <= tol * max(np.abs(want_nb).max(), 1e-3)


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16])
@pytest.mark.parametrize("M,N,K", [(70, 512, 256), (128, 256, 128), (300, 768, 384)])
def test_gemm_hand_ordered_tiles_agree(moe, dtype, M, N, K):
    """The 256 x 256 and the 128 x 256 hand-ordered tiles forced on a plain GEMM (moe_gemm_bias_act_tile): same MFMA
    sequence over K per output element, so bit-identical to each other, and within tolerance of the oracle."""
    rng = np.random.default_rng(M + N + K)
    kind = KIND[dtype]
    A = ob.from_f32(rng.standard_normal((M, K)).astype(np.float32), dtype)
    B = ob.from_f32((rng.standard_normal((N, K)) * 0.1).astype(np.float32), dtype)
    bias = ob.from_f32(rng.standard_normal(N).astype(np.float32), dtype)
    want = ob.to_f32(ob.gemm_bias_act(A, B, bias, dtype, ob.ACT_GELU), dtype)
    outs = []
    for tile in (1, 2):
        outs.append(from_device(moe.gemm_bias_act(to_device(A, kind), to_device(B, kind), to_device(bias, kind), ob.ACT_GELU, tile=tile)))
    assert np.array_equal(outs[0], outs[1])
    tol = {ob.BF16: 1e-2, ob.F16: 1.25e-3}[dtype]
    assert np.abs(ob.to_f32(outs[1], dtype) - want).max() <= tol * np.abs(want).max()


@pytest.mark.parametrize("act", [ob.ACT_RELU, ob.ACT_GELU, ob.ACT_NONE])
@pytest.mark.parametrize("M,N,K", [(1041, 1024, 128), (1280, 1280, 384), (1025, 1536, 1024)])
def test_gemm_large_tile_vs_oracle(moe, M, N, K, act):
    """Shapes that take the 256 x 256 tile with the hand-ordered slab loop (M, N >= 1024, N % 256 = 0, K % 128 = 0):
    the shortest K it accepts, a ragged last row block, bias on and off."""
    rng = np.random.default_rng(M + N + K)
    A = ob.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    B = ob.f32_to_bf16((rng.standard_normal((N, K)) * 0.1).astype(np.float32))
    bias = ob.f32_to_bf16(rng.standard_normal(N).astype(np.float32))
    for b in (bias, None):
        want = ob.to_f32(ob.gemm_bias_act(A, B, b, ob.BF16, act), ob.BF16)
        got = ob.to_f32(from_device(moe.gemm_bias_act(to_device(A, "bf16"), to_device(B, "bf16"),
                                                      None if b is None else to_device(b, "bf16"), act)), ob.BF16)
        assert got.shape == want.shape
        assert np.abs(got - want).max() <= 1e-2 * np.abs(want).max()


def test_gemm_rejects_shapes_it_has_no_kernel_for(moe):
    import torch
    A = torch.zeros(4, 40, device="cuda"); B = torch.zeros(4, 40, device="cuda")
    with pytest.raises(moe.MoEError) as e:
        moe.gemm_bias_act(A, B, None, ob.ACT_RELU)
    assert e.value.status == 2


# ---------------------------------------------------------------- combine (reference Combine contract)
@pytest.mark.parametrize("dtype", [ob.F32, ob.BF16])
def test_combine_reference_identity_case(moe, dtype):
    """hostCombine (combine.cuh:220-231): identity indices, inputs[i][j] = i + 1."""
    M, N = 128, 64
    y = np.repeat(np.arange(1, M + 1, dtype=np.float32)[:, None], N, axis=1)
    kind = "f32" if dtype == ob.F32 else "bf16"
    yy = y if dtype == ob.F32 else ob.f32_to_bf16(y)
    rows = np.arange(M, dtype=np.int32)[:, None]
    out = moe.combine(to_device(yy, kind), to_device(rows, "i32"), to_device(np.ones((M, 1), np.float32), "f32"))
    assert np.array_equal(ob.to_f32(from_device(out), dtype), y)


@pytest.mark.parametrize("dtype,S,k,H", [(ob.F32, 50, 3, 64), (ob.BF16, 333, 6, 2048), (ob.BF16, 64, 8, 7168),
                                         (ob.F16, 200, 2, 1024)])
def test_combine_vs_oracle(moe, dtype, S, k, H):
    rng = np.random.default_rng(S)
    A = S * k
    y = rng.standard_normal((A, H)).astype(np.float32)
    rows = rng.permutation(A).astype(np.int32).reshape(S, k)
    rows[::5, 0] = -1
    rows[3, :] = -1
    w = rng.random((S, k)).astype(np.float32)
    kind = KIND[dtype]
    yy = ob.from_f32(y, dtype)
    want = ob.to_f32(ob.combine(yy, rows, w, H, dtype), dtype)
    got = ob.to_f32(from_device(moe.combine(to_device(yy, kind), to_device(rows, "i32"), to_device(w, "f32"))), dtype)
    tol = {ob.F32: 1e-6, ob.BF16: 2.0 ** -8, ob.F16: 2.0 ** -11}[dtype]
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
    assert (got[3] == 0).all()


# ---------------------------------------------------------------- gate: logits bit-exact, top-k exact
GATE_CASES = [
    ob.Cfg(S=128, H=256, I=64, E=8, k=1, dtype=ob.F32, norm_topk=0),
    ob.Cfg(S=77, H=64, I=64, E=3, k=2, dtype=ob.F32),
    ob.Cfg(S=130, H=1088, I=64, E=64, k=6, dtype=ob.BF16, zipf_bias=True),
    ob.Cfg(S=64, H=7168, I=128, E=256, k=8, dtype=ob.BF16, gate_fn=ob.GATE_SIGMOID),
    ob.Cfg(S=33, H=4096, I=64, E=300, k=16, dtype=ob.BF16, norm_topk=0),
    ob.Cfg(S=1000, H=2048, I=64, E=16, k=2, dtype=ob.BF16),
    ob.Cfg(S=300, H=1536, I=64, E=40, k=4, dtype=ob.F16),
    ob.Cfg(S=20000, H=512, I=64, E=32, k=2, dtype=ob.F16),     # many pairs: the kernel that keeps token rows in registers
    ob.Cfg(S=50, H=128, I=64, E=5, k=2, dtype=ob.TF32),
    ob.Cfg(S=77, H=512, I=64, E=5, k=2, dtype=ob.BF16, zipf_bias=True),      # ragged token and expert tiles of the matrix-core kernel
    ob.Cfg(S=4100, H=1024, I=64, E=8, k=2, dtype=ob.F16),                     # its 16-token x 8-expert arrangement
]


# mfma: the logits kernel on the matrix cores forced on / off (it takes 16-bit layers with H % 512 = 0 only; elsewhere
# the knob changes nothing) -- every kernel must produce the oracle's bit patterns
@pytest.mark.parametrize("mfma", [0, 1], ids=["valu", "mfma"])
@pytest.mark.parametrize("cfg", GATE_CASES, ids=lambda c: "S%d_H%d_E%d_k%d_d%d" % (c.S, c.H, c.E, c.k, c.dtype))
def test_gate_vs_oracle(moe, cfg, mfma):
    inp = ob.make_inputs(cfg, seed=7, router_only=True)
    want = ob.route(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), options={"gate_mfma": mfma})
    dev = upload_inputs(cfg, inp)
    idx, w, logits = layer.gate(dev["x"], dev["gate_w"], dev.get("gate_bias"), want_logits=True)
    assert np.array_equal(bits(from_device(logits)), bits(want["logits"]))      # fp32 bit patterns
    assert np.array_equal(from_device(idx), want["topk_idx"])
    assert np.abs(from_device(w) - want["topk_w"]).max() <= 2e-6
    layer.close()


def test_topk_ties_go_to_lower_index(moe):
    """All-equal logits (zero activations): the selection must be experts 0..k-1 in order."""
    import torch
    cfg = ob.Cfg(S=16, H=64, I=64, E=70, k=5, dtype=ob.BF16)
    layer = moe.MoELayer(product_config(cfg))
    x = torch.zeros(cfg.S, cfg.H, dtype=torch.bfloat16, device="cuda")
    gw = torch.ones(cfg.E, cfg.H, dtype=torch.bfloat16, device="cuda")
    idx, w = layer.gate(x, gw)
    assert np.array_equal(from_device(idx), np.tile(np.arange(5, dtype=np.int32), (cfg.S, 1)))
    assert np.allclose(from_device(w), 0.2)
    layer.close()


# ---------------------------------------------------------------- slot assignment: integer, bit-exact
def random_topk(rng, S, E, k, skew):
    p = np.arange(1, E + 1, dtype=np.float64) ** -skew
    p /= p.sum()
    return np.stack([rng.choice(E, size=k, replace=False, p=p) for _ in range(S)]).astype(np.int32)


@pytest.mark.parametrize("S,E,k,drop,cf,skew", [
    (128, 8, 1, 1, 1.0, 0.0), (1, 1, 1, 0, 1.0, 0.0), (257, 3, 2, 1, 0.5, 1.0), (4096, 16, 2, 1, 1.25, 0.3),
    (3000, 64, 6, 1, 1.0, 1.1), (64, 256, 8, 0, 1.0, 0.0), (1000, 300, 16, 1, 2.0, 0.5), (5000, 2, 1, 0, 1.0, 3.0),
])
def test_route_vs_oracle(moe, S, E, k, drop, cf, skew):
    rng = np.random.default_rng(S + E)
    idx = random_topk(rng, S, E, k, skew)
    cfg = ob.Cfg(S=S, H=64, I=64, E=E, k=k, dtype=ob.BF16, drop=drop, capacity_factor=cf)
    want = ob.route_slots(idx, E, drop, cfg.capacity)
    layer = moe.MoELayer(product_config(cfg))
    got = layer.route(to_device(idx, "i32"))
    for key in ("slot", "expert_count", "expert_offset", "token_indices", "pair_row"):
        assert np.array_equal(from_device(got[key]), want[key]), key
    layer.close()


def test_route_every_token_to_one_expert(moe):
    cfg = ob.Cfg(S=1000, H=64, I=64, E=4, k=1, dtype=ob.BF16, drop=1, capacity_factor=1.0)
    idx = np.full((1000, 1), 2, np.int32)
    want = ob.route_slots(idx, 4, 1, cfg.capacity)
    layer = moe.MoELayer(product_config(cfg))
    got = layer.route(to_device(idx, "i32"))
    assert np.array_equal(from_device(got["slot"]), want["slot"])
    assert list(from_device(got["expert_count"])) == [0, 0, 250, 0]
    layer.close()


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5"])
def test_full_size_routing_matches_golden_digests(moe, name):
    """Gate + slots at the full BASELINE sizes against the committed digests and the oracle."""
    want_d = json.load(open(os.path.join(GOLDEN, "routing_digests.json")))[name]
    cfg = ob.BASELINE[name]
    inp = ob.make_inputs(cfg, want_d["seed"], router_only=True)
    layer = moe.MoELayer(product_config(cfg.scaled(I=128)))      # I does not enter the routing
    dev = upload_inputs(cfg, inp)
    idx, w, logits = layer.gate(dev["x"], dev["gate_w"], dev.get("gate_bias"), want_logits=True)
    r = layer.route(idx)
    sha = lambda a: hashlib.sha256(np.ascontiguousarray(from_device(a)).tobytes()).hexdigest()
    assert sha(logits) == want_d["logits_sha256"]
    assert sha(idx) == want_d["topk_idx_sha256"]
    assert sha(r["slot"]) == want_d["slot_sha256"]
    assert [int(v) for v in from_device(r["expert_count"])] == want_d["expert_count"]
    want = ob.route(cfg, inp)
    assert np.array_equal(from_device(r["token_indices"]), want["token_indices"])
    assert np.abs(from_device(w) - want["topk_w"]).max() <= 2e-6
    layer.close()


@pytest.mark.parametrize("src", ["f32", "bf16"])
def test_quant_block128_bit_exact(moe, src):
    """The GPU quantiser against the oracle's, codes and scales bit for bit, including the awkward values."""
    import torch
    rng = np.random.default_rng(17)
    w = (rng.standard_normal((3, 256, 384)) * 0.02).astype(np.float32)
    w[0, :128, :128] = 0.0                                   # an all-zero block: scale 1, codes 0
    w[1, 5, 7] = 3.0                                         # one dominant value: the rest lands in the subnormals
    w[1, 130, 200] = -np.float32(1e-30)
    w[2, :128, 128:256] *= np.float32(1e-20)                 # tiny magnitudes, still scaled to the full range
    # exact ties of the 3-bit mantissa after scaling by 1/448 * 448 = 1: block maximum 448 keeps scale 1
    w[2, 128:, 256:] = 0.0
    w[2, 128, 256] = 448.0
    w[2, 129, 256:264] = np.array([1.0625, 1.1875, 17.0, 19.0, 0.0009765625, 0.0029296875, 447.9, 464.0], np.float32)
    if src == "bf16":
        bits = ob.f32_to_bf16(w)
        w = ob.bf16_to_f32(bits)
        dev = to_device(bits, "bf16")
    else:
        dev = to_device(w, "f32")
    want_q, want_s = ob.quant_block128(w)
    q, s = moe.quantize_block128(dev)
    torch.cuda.synchronize()
    assert np.array_equal(s.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    assert np.array_equal(q.cpu().numpy(), want_q)


@pytest.mark.parametrize("name", ["C1", "C4", "C5"])
def test_router_stats_vs_oracle(moe, name):
    """moe_router_stats on the GPU's own logits and choices against the oracle's fp64 sums (fp32 results, 1e-6)."""
    import torch
    cfg = ob.BASELINE[name]
    small = ob.Cfg(S=min(cfg.S, 2048), H=min(cfg.H, 512), I=256, E=cfg.E, k=cfg.k, act=cfg.act, dtype=ob.BF16,
                   gate_fn=cfg.gate_fn, norm_topk=cfg.norm_topk, drop=0, zipf_bias=cfg.zipf_bias)
    inp = ob.make_inputs(small, seed=13, router_only=True)
    dev = upload_inputs(small, inp)
    layer = moe.MoELayer(product_config(small))
    idx, _, logits = layer.gate(dev["x"], dev["gate_w"], dev.get("gate_bias"), want_logits=True)
    got = layer.router_stats(logits, idx)
    torch.cuda.synchronize()
    want = ob.router_stats(logits.cpu().numpy(), idx.cpu().numpy(), small.gate_fn)
    assert np.allclose(got["mean_prob"].cpu().numpy(), want["mean_prob"], rtol=1e-6, atol=1e-9)
    assert np.array_equal(got["load"].cpu().numpy(), want["load"])
    assert abs(float(got["aux_loss"].cpu()[0]) - want["aux_loss"]) <= 1e-6 * max(1.0, abs(want["aux_loss"]))
    again = layer.router_stats(logits, idx)
    torch.cuda.synchronize()
    assert torch.equal(again["mean_prob"], got["mean_prob"]) and torch.equal(again["aux_loss"], got["aux_loss"])
    layer.close()
