"""GPU parity of the backward building blocks (batched transpose, grouped product over packed expert rows, per-expert
weight gradient), called through the C ABI, against the CPU oracle."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, to_device

pytestmark = pytest.mark.gpu
KIND = {ob.BF16: "bf16", ob.F16: "f16", ob.F32: "f32"}


@pytest.fixture(scope="module")
def moe():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import cuplayground_amd
    cuplayground_amd.load_library()
    return cuplayground_amd


def routed_case(S, H, I, E, k, dtype, seed, drop=1, cf=1.0, skew=0.0):
    """A layer shape with a real routing result from the oracle: counts and offsets as moe_route writes them."""
    cfg = ob.Cfg(S=S, H=H, I=I, E=E, k=k, dtype=dtype, act=ob.ACT_GELU, drop=drop, capacity_factor=cf, norm_topk=1)
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((S, E)).astype(np.float32) + skew * np.arange(E, dtype=np.float32)
    idx, _ = ob.topk(logits, k, cfg.gate_fn, cfg.norm_topk)
    r = ob.route_slots(idx, E, cfg.drop, cfg.capacity)
    return cfg, rng, r["expert_count"], r["expert_offset"]


def operands(rng, R, E, N, K, dtype):
    a = ob.from_f32(rng.standard_normal((R, K)).astype(np.float32), dtype)
    dy = ob.from_f32(rng.standard_normal((R, N)).astype(np.float32), dtype)
    w = ob.from_f32((rng.standard_normal((E, N, K)) * 0.1).astype(np.float32), dtype)
    bias = ob.from_f32(rng.standard_normal((E, N)).astype(np.float32), dtype)
    return a, dy, w, bias


@pytest.mark.parametrize("shape", [(1, 5, 7), (3, 64, 64), (2, 130, 257), (4, 1000, 72), (2, 8, 264), (3, 200, 1032)])
@pytest.mark.parametrize("elem", [2, 4])
def test_transpose_is_exact(moe, shape, elem):
    rng = np.random.default_rng(sum(shape))
    a = rng.integers(0, 2 ** (8 * elem) - 1, shape, dtype=np.uint64).astype(np.uint16 if elem == 2 else np.uint32)
    t = moe.api.transpose(to_device(a.view(np.int16 if elem == 2 else np.int32), "i32"))
    assert np.array_equal(from_device(t).view(a.dtype), a.transpose(0, 2, 1))


CASES = [  # S, H, I, E, k, capacity factor, router skew
    (256, 256, 512, 8, 2, 1.0, 0.0),
    (512, 128, 320, 4, 1, 2.0, 0.7),        # skewed: one expert takes most rows, one may stay empty
    (2048, 512, 1024, 4, 2, 1.25, 0.0),     # 256-row blocks in the grouped product
    (1024, 1024, 1024, 2, 2, 2.0, 0.0),     # 256 x 256 tiles in the weight gradient as well
]


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16, ob.F32])
@pytest.mark.parametrize("case", CASES)
def test_expert_gemm_vs_oracle(moe, case, dtype):
    S, H, I, E, k, cf, skew = case
    cfg, rng, count, offset = routed_case(S, H, I, E, k, dtype, seed=S + E, cf=cf, skew=skew)
    layer = moe.MoELayer(product_config(cfg))
    kind = KIND[dtype]
    dcount, doffset = to_device(count, "i32"), to_device(offset, "i32")
    for (N, K, act, with_bias) in ((I, H, ob.ACT_GELU, True), (H, I, ob.ACT_NONE, False), (H, I, ob.ACT_RELU, True)):
        a, _, w, bias = operands(rng, S * k, E, N, K, dtype)
        want = ob.to_f32(ob.expert_gemm(a, w, bias if with_bias else None, count, offset, dtype, act), dtype)
        got = layer.expert_gemm(to_device(a, kind), to_device(w, kind), to_device(bias, kind) if with_bias else None,
                                dcount, doffset, act)
        got = ob.to_f32(from_device(got), dtype)
        kept = int(count.sum())
        assert max_rel_err(got[:kept], want[:kept]) <= OUT_TOL[dtype]
        assert not got[kept:].any()            # rows of no expert are not written (the output started as zeros)


def test_fp32_products_on_the_matrix_core_tile_and_on_the_vector_tile(moe):
    """fp32 layers: the grouped product and the weight gradient of a shape that takes the 128 x 128 matrix-core tile,
    and the same calls held on the 64 x 64 vector-ALU tile (a handle created with the option f32_tile = 0).  Both within the fp32 tolerance of the
    oracle; their sums run in different orders, so the results are not the same bits -- which shows both ran."""
    S, H, I, E, k, cf, skew = CASES[2]
    dtype = ob.F32
    cfg, rng, count, offset = routed_case(S, H, I, E, k, dtype, seed=79, cf=cf, skew=0.3)
    layers = {"0": moe.MoELayer(product_config(cfg), options={"f32_tile": 0}), None: moe.MoELayer(product_config(cfg), options={})}
    a, dy, w, bias = operands(rng, S * k, E, I, H, dtype)
    want = ob.expert_gemm(a, w, bias, count, offset, dtype, ob.ACT_GELU)
    want_dw = ob.expert_wgrad(dy, a, count, offset, dtype)
    kept = int(count.sum())
    dev = [to_device(v, "f32") for v in (a, dy, w, bias)] + [to_device(count, "i32"), to_device(offset, "i32")]
    outs, grads = {}, {}
    for knob in ("0", None):
        layer = layers[knob]
        outs[knob] = from_device(layer.expert_gemm(dev[0], dev[2], dev[3], dev[4], dev[5], ob.ACT_GELU))
        grads[knob] = from_device(layer.expert_wgrad(dev[1], dev[0], dev[4], dev[5]))
        assert max_rel_err(outs[knob][:kept], want[:kept]) <= OUT_TOL[dtype]
        for e in range(E):
            if count[e] > 0:
                assert max_rel_err(grads[knob][e], want_dw[e]) <= OUT_TOL[dtype], e
    assert not np.array_equal(outs["0"][:kept], outs[None][:kept])
    assert not np.array_equal(grads["0"], grads[None])


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16])
def test_grouped_product_tiles_agree(moe, dtype):
    """The 128 x 128, 256 x 256 and 128 x 256 tiles forced on one grouped product (option grouped_tile): the two
    hand-ordered ones accumulate every output element with the same MFMA sequence and must agree bit for bit; the
    compiler-ordered 128 x 128 tile only within the tolerance."""
    S, H, I, E, k, cf, skew = CASES[2]
    cfg, rng, count, offset = routed_case(S, H, I, E, k, dtype, seed=77, cf=cf, skew=0.3)
    kind = KIND[dtype]
    a, _, w, bias = operands(rng, S * k, E, I, H, dtype)
    want = ob.to_f32(ob.expert_gemm(a, w, bias, count, offset, dtype, ob.ACT_GELU), dtype)
    outs = {}
    for tile in ("0", "1", "2"):
        layer = moe.MoELayer(product_config(cfg), options={"grouped_tile": int(tile)})
        got = layer.expert_gemm(to_device(a, kind), to_device(w, kind), to_device(bias, kind), to_device(count, "i32"),
                                to_device(offset, "i32"), ob.ACT_GELU)
        outs[tile] = from_device(got)
        kept = int(count.sum())
        assert max_rel_err(ob.to_f32(outs[tile], dtype)[:kept], want[:kept]) <= OUT_TOL[dtype]
    assert np.array_equal(outs["1"], outs["2"])


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16, ob.F32])
@pytest.mark.parametrize("case", CASES)
def test_data_gradient_is_the_grouped_product_with_the_transposed_weight(moe, case, dtype):
    """dX = dY . W: the oracle works on numpy's transpose, the product on moe_transpose's."""
    S, H, I, E, k, cf, skew = case
    cfg, rng, count, offset = routed_case(S, H, I, E, k, dtype, seed=3 * S + E, cf=cf, skew=skew)
    layer = moe.MoELayer(product_config(cfg))
    kind = KIND[dtype]
    _, dy, w, _ = operands(rng, S * k, E, H, I, dtype)           # down projection: y [*, H] = h [*, I] . w[e]^T, w [E, H, I]
    wT = np.ascontiguousarray(w.transpose(0, 2, 1))              # [E, I, H]
    want = ob.to_f32(ob.expert_gemm(dy, wT, None, count, offset, dtype, ob.ACT_NONE), dtype)
    dwT = moe.api.transpose(to_device(w, kind))
    assert np.array_equal(from_device(dwT), wT)
    got = layer.expert_gemm(to_device(dy, kind), dwT, None, to_device(count, "i32"), to_device(offset, "i32"))
    kept = int(count.sum())
    assert max_rel_err(ob.to_f32(from_device(got), dtype)[:kept], want[:kept]) <= OUT_TOL[dtype]


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16, ob.F32])
@pytest.mark.parametrize("case", CASES)
def test_weight_gradient_vs_oracle(moe, case, dtype):
    S, H, I, E, k, cf, skew = case
    cfg, rng, count, offset = routed_case(S, H, I, E, k, dtype, seed=5 * S + E, cf=cf, skew=skew)
    layer = moe.MoELayer(product_config(cfg))
    kind = KIND[dtype]
    dcount, doffset = to_device(count, "i32"), to_device(offset, "i32")
    for (N, K) in ((H, I), (I, H)):
        a, dy, _, _ = operands(rng, S * k, E, N, K, dtype)
        want = ob.to_f32(ob.expert_wgrad(dy, a, count, offset, dtype), dtype)
        got = ob.to_f32(from_device(layer.expert_wgrad(to_device(dy, kind), to_device(a, kind), dcount, doffset)), dtype)
        for e in range(E):
            if count[e] == 0:
                assert not got[e].any()
            else:
                assert max_rel_err(got[e], want[e]) <= OUT_TOL[dtype], (e, int(count[e]))


def test_empty_experts_and_second_call_reuse_scratch(moe):
    """All rows on one expert, then a different split through the same layer: stale scratch must not leak."""
    dtype, kind = ob.BF16, "bf16"
    S, H, I, E = 256, 128, 256, 4
    cfg = ob.Cfg(S=S, H=H, I=I, E=E, k=1, dtype=dtype, act=ob.ACT_RELU, drop=0)
    layer = moe.MoELayer(product_config(cfg))
    rng = np.random.default_rng(9)
    a, dy, _, _ = operands(rng, S, E, H, I, dtype)
    for count in ([0, S, 0, 0], [100, 0, 29, 127], [0, 0, 0, 0]):
        count = np.asarray(count, np.int32)
        offset = np.concatenate([[0], np.cumsum(count)[:-1]]).astype(np.int32)
        want = ob.to_f32(ob.expert_wgrad(dy, a, count, offset, dtype), dtype)
        got = ob.to_f32(from_device(layer.expert_wgrad(to_device(dy, kind), to_device(a, kind),
                                                       to_device(count, "i32"), to_device(offset, "i32"))), dtype)
        assert np.abs(got - want).max() <= OUT_TOL[dtype] * max(np.abs(want).max(), 1.0)


def test_unsupported_layers_and_bad_arguments_are_refused(moe):
    import torch
    cfg = ob.Cfg(S=128, H=128, I=256, E=4, k=1, dtype=ob.FP8, act=ob.ACT_RELU, drop=0)
    layer = moe.MoELayer(product_config(cfg))
    with pytest.raises(moe.MoEError) as e:
        layer.backward_scratch()
    assert e.value.status == 2                    # e4m3 layers have no backward kernels
    cfg = ob.Cfg(S=128, H=128, I=256, E=4, k=1, dtype=ob.BF16, act=ob.ACT_RELU, drop=0)
    layer = moe.MoELayer(product_config(cfg))
    z = torch.zeros(128, 192, dtype=torch.bfloat16, device="cuda")
    w = torch.zeros(4, 256, 192, dtype=torch.bfloat16, device="cuda")
    cnt = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(moe.MoEError) as e:        # (N, K) = (256, 192) is no projection of this layer
        layer.expert_gemm(z, w, None, cnt, cnt)
    assert e.value.status == 4


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16, ob.F32])
@pytest.mark.parametrize("act", [ob.ACT_RELU, ob.ACT_GELU, ob.ACT_SWIGLU])
def test_activation_backward_vs_oracle(moe, act, dtype):
    cfg = ob.Cfg(S=300, H=128, I=320, E=4, k=2, dtype=dtype, act=act, drop=0)
    layer = moe.MoELayer(product_config(cfg))
    kind = KIND[dtype]
    rng = np.random.default_rng(31 + act)
    rows = cfg.S * cfg.k - 7                                   # fewer rows than the buffers hold
    u = ob.from_f32(rng.standard_normal((cfg.S * cfg.k, cfg.I)).astype(np.float32) * 2, dtype)
    g = ob.from_f32(rng.standard_normal((cfg.S * cfg.k, cfg.I)).astype(np.float32) * 2, dtype)
    dh = ob.from_f32(rng.standard_normal((cfg.S * cfg.k, cfg.I)).astype(np.float32), dtype)
    sw = act == ob.ACT_SWIGLU
    want_du, want_dg = ob.act_backward(dh[:rows], u[:rows], g[:rows] if sw else None, dtype, act)
    du, dg = layer.act_backward(to_device(dh, kind)[:rows], to_device(u, kind)[:rows], to_device(g, kind)[:rows] if sw else None)
    # library exp / erf against libm: an output ulp at most
    tol = OUT_TOL[dtype]
    assert max_rel_err(ob.to_f32(from_device(du), dtype), ob.to_f32(want_du, dtype)) <= tol
    if sw:
        assert max_rel_err(ob.to_f32(from_device(dg), dtype), ob.to_f32(want_dg, dtype)) <= tol
    else:
        assert dg is None


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16, ob.F32])
@pytest.mark.parametrize("act", [ob.ACT_GELU, ob.ACT_SWIGLU])
def test_activation_backward_does_not_depend_on_alignment(moe, act, dtype):
    """16 bytes per operand and thread where every pointer allows it, one element at a time where not: the same bits
    either way, and nothing written in front of the first element or past the last."""
    import torch
    cfg = ob.Cfg(S=300, H=128, I=320, E=4, k=2, dtype=dtype, act=act, drop=0)
    layer = moe.MoELayer(product_config(cfg))
    kind = KIND[dtype]
    rng = np.random.default_rng(77 + act)
    rows = cfg.S * cfg.k - 7
    n = rows * cfg.I
    sw = act == ob.ACT_SWIGLU
    host = {name: ob.from_f32(rng.standard_normal(n).astype(np.float32) * 2, dtype) for name in ("dh", "u", "g")}

    def run(shift):
        """Operands and results `shift` elements into their buffers; a guard value behind each result."""
        dev = {}
        for name, v in host.items():
            buf = torch.zeros(n + 16, dtype=layer.act_dtype, device="cuda")
            buf[shift:shift + n] = to_device(v, kind)
            dev[name] = buf[shift:shift + n].view(rows, cfg.I)
        outs = [torch.full((n + 16,), 7.0, dtype=layer.act_dtype, device="cuda") for _ in range(2)]
        du, dg = (o[shift:shift + n].view(rows, cfg.I) for o in outs)
        layer.act_backward(dev["dh"], dev["u"], dev["g"] if sw else None, du=du, dg=dg if sw else None)
        torch.cuda.synchronize()
        for o in outs[:2 if sw else 1]:
            assert (o[:shift] == 7.0).all() and (o[shift + n:] == 7.0).all()
        return from_device(du.contiguous()), from_device(dg.contiguous()) if sw else None

    du0, dg0 = run(0)
    du1, dg1 = run(1)
    assert np.array_equal(du0, du1)
    want_du, want_dg = ob.act_backward(host["dh"].reshape(rows, -1), host["u"].reshape(rows, -1),
                                       host["g"].reshape(rows, -1) if sw else None, dtype, act)
    assert max_rel_err(ob.to_f32(du0, dtype), ob.to_f32(want_du, dtype)) <= OUT_TOL[dtype]
    if sw:
        assert np.array_equal(dg0, dg1)
        assert max_rel_err(ob.to_f32(dg0, dtype), ob.to_f32(want_dg, dtype)) <= OUT_TOL[dtype]
    layer.close()


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16, ob.F32])
def test_bias_gradient_is_bit_exact(moe, dtype):
    """One thread per column adds the rows in ascending order, as the oracle does: the same fp32 sums, bit for bit."""
    S, H, I, E, k, cf, skew = CASES[1]
    cfg, rng, count, offset = routed_case(S, H, I, E, k, dtype, seed=91, cf=cf, skew=skew)
    layer = moe.MoELayer(product_config(cfg))
    kind = KIND[dtype]
    for N in (H, I):
        dy = ob.from_f32(rng.standard_normal((S * k, N)).astype(np.float32), dtype)
        got = from_device(layer.bias_grad(to_device(dy, kind), to_device(count, "i32"), to_device(offset, "i32")))
        assert np.array_equal(got, ob.bias_grad(dy, count, offset, dtype))


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16, ob.F32])
def test_combine_backward_vs_oracle(moe, dtype):
    cfg = ob.Cfg(S=257, H=320, I=128, E=5, k=3, dtype=dtype, act=ob.ACT_RELU, drop=1, capacity_factor=0.8)
    rng = np.random.default_rng(41)
    logits = rng.standard_normal((cfg.S, cfg.E)).astype(np.float32)
    idx, w = ob.topk(logits, cfg.k, cfg.gate_fn, cfg.norm_topk)
    r = ob.route_slots(idx, cfg.E, cfg.drop, cfg.capacity)
    assert (r["pair_row"] < 0).any()
    layer = moe.MoELayer(product_config(cfg))
    kind = KIND[dtype]
    y = ob.from_f32(rng.standard_normal((cfg.S * cfg.k, cfg.H)).astype(np.float32), dtype)
    dout = ob.from_f32(rng.standard_normal((cfg.S, cfg.H)).astype(np.float32), dtype)
    want_dy, want_dw = ob.combine_backward(dout, y, r["pair_row"], w, dtype)
    dy, dw = layer.combine_backward(to_device(dout, kind), to_device(y, kind), to_device(r["pair_row"], "i32"), to_device(w, "f32"))
    if dtype in (ob.BF16, ob.F32):
        assert np.array_equal(from_device(dy), want_dy)        # one multiplication and one rounding per element
    else:   # fp16: the compiler multiplies and narrows in one mixed-precision instruction (one rounding), the oracle
        # rounds the fp32 product first; on near-ties they differ by one fp16 ulp
        got, ref = ob.to_f32(from_device(dy), dtype), ob.to_f32(want_dy, dtype)
        assert np.abs(got - ref).max() <= 2.0 ** -10 * np.abs(ref).max()
        assert (from_device(dy) != want_dy).mean() < 1e-3
    assert np.abs(from_device(dw) - want_dw).max() <= 1e-5 * max(np.abs(want_dw).max(), 1.0)
    assert not from_device(dw)[r["pair_row"] < 0].any()


FUSED_CASES = [  # S, H, I, E, k, capacity factor, router skew, option grouped_tile (None: the library's choice)
    (2048, 512, 1024, 4, 2, 1.25, 0.0, None),    # 256-row blocks
    (2048, 512, 1024, 4, 2, 1.25, 0.3, 2),       # the same rows on 128-row blocks
    (512, 128, 256, 4, 1, 2.0, 0.7, None),       # few rows per expert, ragged last blocks, an expert that may stay empty
    (700, 256, 512, 3, 2, 1.0, 0.0, 1),          # 256-row blocks forced on few rows
]


@pytest.mark.parametrize("dtype", [ob.BF16, ob.F16])
@pytest.mark.parametrize("act", [ob.ACT_RELU, ob.ACT_GELU, ob.ACT_SWIGLU])
@pytest.mark.parametrize("case", FUSED_CASES)
def test_fused_activation_backward_is_the_two_call_chain(moe, case, act, dtype):
    """moe_expert_gemm_act_backward against moe_expert_gemm (no activation) followed by moe_act_backward: the product is
    rounded to the storage type before the derivative in both, and both inline the same derivative, so the kept rows
    agree bit for bit; against the oracle's chain within the layer's tolerance."""
    S, H, I, E, k, cf, skew, tile = case
    cfg, rng, count, offset = routed_case(S, H, I, E, k, dtype, seed=5 + act, cf=cf, skew=skew)
    cfg = cfg.scaled(act=act)
    kind = KIND[dtype]
    layer = moe.MoELayer(product_config(cfg), options={} if tile is None else {"grouped_tile": tile})
    assert layer.fused_act_backward
    R = S * k
    kept = int(count.sum())
    assert 0 < kept <= R
    dy, _, w_t, _ = operands(rng, R, E, I, H, dtype)              # dy [R, H] is the product's left operand; w_t [E, I, H]
    u = ob.from_f32(rng.standard_normal((R, I)).astype(np.float32) * 2, dtype)
    sw = act == ob.ACT_SWIGLU
    g = ob.from_f32(rng.standard_normal((R, I)).astype(np.float32) * 2, dtype) if sw else None
    d = {n: to_device(v, kind) for n, v in (("dy", dy), ("w", w_t), ("u", u))}
    dg_in = to_device(g, kind) if sw else None
    cnt, off = to_device(count, "i32"), to_device(offset, "i32")
    du, dg = layer.expert_gemm_act_backward(d["dy"], d["w"], d["u"], dg_in, cnt, off)
    dh = layer.expert_gemm(d["dy"], d["w"], None, cnt, off, ob.ACT_NONE)
    du2, dg2 = layer.act_backward(dh[:kept], d["u"][:kept], dg_in[:kept] if sw else None)
    assert np.array_equal(from_device(du)[:kept], from_device(du2))
    assert not from_device(du)[kept:].any()                       # rows of no expert are not written
    want_dh = ob.expert_gemm(dy, w_t, None, count, offset, dtype, ob.ACT_NONE)
    want_du, want_dg = ob.act_backward(want_dh[:kept], u[:kept], g[:kept] if sw else None, dtype, act)
    assert max_rel_err(ob.to_f32(from_device(du), dtype)[:kept], ob.to_f32(want_du, dtype)) <= OUT_TOL[dtype]
    if sw:
        assert np.array_equal(from_device(dg)[:kept], from_device(dg2))
        assert not from_device(dg)[kept:].any()
        assert max_rel_err(ob.to_f32(from_device(dg), dtype)[:kept], ob.to_f32(want_dg, dtype)) <= OUT_TOL[dtype]
    else:
        assert dg is None and dg2 is None
    layer.close()


def test_fused_activation_backward_says_where_it_does_not_exist(moe):
    import torch
    base = ob.Cfg(S=256, H=128, I=256, E=4, k=1, dtype=ob.BF16, act=ob.ACT_SWIGLU, drop=0)
    cases = [
        (base, {}, True),
        (base, {"grouped_tile": 0}, False),                       # the 128 x 128 tile has no such epilogue
        (base.scaled(I=384), {}, False),                          # 384 columns are no multiple of the tile's 256
        (base.scaled(H=192), {}, False),                          # the slab loop takes 128 elements of the sum at a time
        (base.scaled(dtype=ob.F32), {}, False),
    ]
    for cfg, opts, want in cases:
        layer = moe.MoELayer(product_config(cfg), options=opts)
        assert layer.fused_act_backward == want, (cfg.H, cfg.I, cfg.dtype, opts)
        if not want:
            dt = layer.act_dtype
            z = lambda *s: torch.zeros(*s, dtype=dt, device="cuda")
            cnt = torch.zeros(cfg.E, dtype=torch.int32, device="cuda")
            with pytest.raises(moe.MoEError) as e:
                layer.expert_gemm_act_backward(z(cfg.S, cfg.H), z(cfg.E, cfg.I, cfg.H), z(cfg.S, cfg.I), z(cfg.S, cfg.I), cnt, cnt)
            assert e.value.status == 2
        layer.close()
    layer = moe.MoELayer(product_config(base))
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device="cuda")
    cnt = torch.zeros(base.E, dtype=torch.int32, device="cuda")
    with pytest.raises(moe.MoEError) as e:                        # a SwiGLU layer needs the gate's rows
        layer.expert_gemm_act_backward(z(256, 128), z(4, 256, 128), z(256, 256), None, cnt, cnt)
    assert e.value.status == 4
    with pytest.raises(moe.MoEError) as e:                        # (N, K) = (128, 256) is the up projection's gradient
        layer.expert_gemm_act_backward(z(256, 256), z(4, 128, 256), z(256, 128), z(256, 128), cnt, cnt)
    assert e.value.status == 4
    layer.close()
