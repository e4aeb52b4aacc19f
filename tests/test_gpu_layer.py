"""GPU parity of the whole layer (moe_forward through the C ABI) against the CPU oracle."""
import os

import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, upload_inputs
from test_oracle_layer import CASES, dense_mixture

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FFN_TILED, FFN_PERSISTENT = 1, 2
ROUTING_KEYS = ("topk_idx", "slot", "expert_count", "expert_offset", "token_indices")


@pytest.fixture(scope="module")
def moe():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import cuplayground_amd
    cuplayground_amd.load_library()
    return cuplayground_amd


def run_layer(moe, cfg, inp, mode, options=None):
    """options: a dict of moe_options fields; None = the handle moe_create makes (library defaults)."""
    import torch
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, options=options)
    dev = upload_inputs(cfg, inp)
    routing = layer.new_routing()
    out = layer.forward(dev["x"], dev, routing=routing)
    torch.cuda.synchronize()
    layer.task_counts()            # raises if the persistent queue recorded a stalled dependency wait
    res = {k: from_device(v) for k, v in routing.items()}
    res["out"] = from_device(out)
    res["plan"] = layer.plan
    layer.close()
    return res


def check_routing(got, want):
    for key in ROUTING_KEYS:
        assert np.array_equal(got[key], want[key]), key
    assert np.abs(got["topk_w"] - want["topk_w"]).max() <= 2e-6


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
def test_c1_against_golden_fixture(moe, mode):
    cfg = ob.BASELINE["C1"]
    g = np.load(os.path.join(GOLDEN, "c1_layer.npz"))
    got = run_layer(moe, cfg, ob.make_inputs(cfg, 42), mode)
    check_routing(got, g)
    assert max_rel_err(got["out"], g["out"]) <= OUT_TOL[ob.F32]
    assert (got["out"][(g["slot"] < 0).all(axis=1)] == 0).all()


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
@pytest.mark.parametrize("name", sorted(CASES))
def test_small_layers_vs_oracle(moe, name, mode):
    cfg = CASES[name]
    inp = ob.make_inputs(cfg, seed=11, with_bias="bias" in name)
    want = ob.forward(cfg, inp)
    got = run_layer(moe, cfg, inp, mode)
    check_routing(got, want)
    err = max_rel_err(ob.to_f32(got["out"], cfg.act_dtype), ob.to_f32(want["out"], cfg.act_dtype))
    assert err <= OUT_TOL[cfg.dtype], err
    # and against float64 math that shares nothing with the oracle's loops
    ref = dense_mixture(cfg, inp, want)
    assert max_rel_err(ob.to_f32(got["out"], cfg.act_dtype), ref) <= max(OUT_TOL[cfg.dtype], 2e-5)


RAGGED = {
    # rows per expert straddle tile boundaries, some experts get nothing, biases on
    "bf16_gelu_ragged": ob.Cfg(S=700, H=192, I=320, E=5, k=2, act=ob.ACT_GELU, dtype=ob.BF16, drop=1,
                               capacity_factor=1.1),
    "bf16_relu_bias": ob.Cfg(S=300, H=128, I=192, E=3, k=1, act=ob.ACT_RELU, dtype=ob.BF16, norm_topk=0, drop=0),
    "bf16_swiglu_skew": ob.Cfg(S=1500, H=256, I=192, E=64, k=6, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=1,
                               capacity_factor=1.0, zipf_bias=True),
    "bf16_swiglu_bias_dropless": ob.Cfg(S=513, H=320, I=448, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0),
    "f32_swiglu_ragged": ob.Cfg(S=333, H=192, I=320, E=7, k=3, act=ob.ACT_SWIGLU, dtype=ob.F32, drop=1,
                                capacity_factor=0.75),
    "fp8_decode_small": ob.Cfg(S=64, H=512, I=256, E=32, k=8, act=ob.ACT_SWIGLU, dtype=ob.FP8,
                               gate_fn=ob.GATE_SIGMOID, drop=0),
    "fp8_many_rows_bias": ob.Cfg(S=200, H=384, I=384, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8,
                                 gate_fn=ob.GATE_SIGMOID, drop=1, capacity_factor=1.0),
    "fp16_swiglu_skew_bias": ob.Cfg(S=900, H=256, I=320, E=24, k=4, act=ob.ACT_SWIGLU, dtype=ob.F16, drop=1,
                                    capacity_factor=1.0, zipf_bias=True),
    "fp16_relu_ragged": ob.Cfg(S=301, H=192, I=448, E=5, k=2, act=ob.ACT_RELU, dtype=ob.F16, drop=0),
    "tf32_gelu_ragged": ob.Cfg(S=150, H=128, I=192, E=4, k=2, act=ob.ACT_GELU, dtype=ob.TF32, drop=1, capacity_factor=0.8),
    "one_token": ob.Cfg(S=1, H=64, I=64, E=2, k=1, act=ob.ACT_GELU, dtype=ob.BF16, norm_topk=0, drop=0),
    # every expert selected by every token; a single expert; the widest router the kernels take; capacity of one row
    "all_experts_selected": ob.Cfg(S=100, H=64, I=64, E=4, k=4, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0),
    "single_expert": ob.Cfg(S=300, H=128, I=64, E=1, k=1, act=ob.ACT_GELU, dtype=ob.BF16, norm_topk=0, drop=0),
    "many_experts_bias": ob.Cfg(S=128, H=128, I=128, E=512, k=16, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0),
    "capacity_one": ob.Cfg(S=64, H=64, I=128, E=8, k=2, act=ob.ACT_RELU, dtype=ob.BF16, drop=1, capacity_factor=0.05),
    "f32_single_expert_top1": ob.Cfg(S=70, H=64, I=64, E=1, k=1, act=ob.ACT_RELU, dtype=ob.F32, norm_topk=0, drop=0),
}


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
@pytest.mark.parametrize("name", sorted(RAGGED))
def test_ragged_layers_vs_oracle(moe, name, mode):
    cfg = RAGGED[name]
    inp = ob.make_inputs(cfg, seed=3, with_bias="bias" in name)
    want = ob.forward(cfg, inp)
    got = run_layer(moe, cfg, inp, mode)
    check_routing(got, want)
    err = max_rel_err(ob.to_f32(got["out"], cfg.act_dtype), ob.to_f32(want["out"], cfg.act_dtype))
    assert err <= OUT_TOL[cfg.dtype], err
    dead = (want["slot"] < 0).all(axis=1)
    assert (ob.to_f32(got["out"], cfg.act_dtype)[dead] == 0).all()


@pytest.mark.parametrize("name", ["bf16_swiglu_skew", "bf16_gelu_ragged", "fp8_decode_small", "f32_swiglu_ragged"])
def test_task_totals_match_the_reference_bound(moe, name):
    """tasks = sum over experts of tilesM * tilesNx (first GEMM) and tilesM * tilesN (second GEMM)
    (scheduling.cuh:212-222), with tilesM from the routed row counts; the hardware description is sane."""
    import torch
    cfg = RAGGED[name]
    inp = ob.make_inputs(cfg, seed=3)
    want = ob.forward(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT)
    dev = upload_inputs(cfg, inp)
    layer.forward(dev["x"], dev)
    torch.cuda.synchronize()
    t0, t1 = layer.task_counts()
    plan = layer.plan
    tiles_m = sum(-(-int(c) // plan["block_rows"]) for c in want["expert_count"])
    assert t0 == tiles_m * plan["col_tiles_up"] and t1 == tiles_m * plan["col_tiles_down"]
    arch = layer.arch
    assert arch["name"].startswith("gfx950") and arch["wavefront_size"] == 64 and arch["compute_units"] >= 1
    assert arch["persistent_blocks"] >= arch["compute_units"]
    layer.close()


def test_repeat_calls_are_deterministic_and_workspace_is_reusable(moe):
    import torch
    cfg = RAGGED["bf16_swiglu_skew"]
    inp = ob.make_inputs(cfg, seed=3)
    layer = moe.MoELayer(product_config(cfg))
    dev = upload_inputs(cfg, inp)
    a = layer.forward(dev["x"], dev).clone()
    for mode in (FFN_TILED, FFN_PERSISTENT, FFN_PERSISTENT):
        layer.set_ffn_mode(mode)
        b = layer.forward(dev["x"], dev)
        assert torch.equal(a, b)
    layer.close()


def test_argument_errors(moe):
    import torch
    cfg = CASES["bf16_gelu_top2"]
    layer = moe.MoELayer(product_config(cfg))
    dev = upload_inputs(cfg, ob.make_inputs(cfg, seed=11))
    with pytest.raises(moe.MoEError) as e:      # w_gate given for a non-SwiGLU layer
        layer.forward(dev["x"], {**dev, "w_gate": dev["w_up"]})
    assert e.value.status == 4
    with pytest.raises(moe.MoEError) as e:      # scales given for a bf16 layer
        layer.forward(dev["x"], {**dev, "s_up": dev["gate_w"], "s_down": dev["gate_w"], "s_gate": dev["gate_w"]})
    assert e.value.status == 4
    ws = layer.workspace
    layer.workspace = ws[: ws.numel() // 2]
    layer.workspace_bytes = layer.workspace.numel()
    with pytest.raises(moe.MoEError) as e:
        layer.forward(dev["x"], dev)
    assert e.value.status == 3
    layer.close()


LARGE_TILE = {
    # row blocks of 256 with partial tails; full column tiles (hand-ordered slab loop) and ragged ones (general loop)
    "swiglu_bias": ob.Cfg(S=1500, H=256, I=384, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0),
    "gelu_bias_drop": ob.Cfg(S=1300, H=384, I=512, E=3, k=2, act=ob.ACT_GELU, dtype=ob.BF16, drop=1,
                             capacity_factor=0.9),
    "relu_ragged_n": ob.Cfg(S=900, H=320, I=448, E=2, k=1, act=ob.ACT_RELU, dtype=ob.BF16, norm_topk=0, drop=0),
    "swiglu_k_not_128": ob.Cfg(S=800, H=192, I=320, E=3, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0),
    # the shortest K the slab loop takes (two slabs in the down projection), row blocks that are exactly full
    "swiglu_two_slabs": ob.Cfg(S=512, H=256, I=128, E=1, k=1, act=ob.ACT_SWIGLU, dtype=ob.BF16, norm_topk=0, drop=0),
    "fp16_swiglu_bias": ob.Cfg(S=1400, H=256, I=256, E=3, k=2, act=ob.ACT_SWIGLU, dtype=ob.F16, drop=0),
    "fp16_gelu_drop": ob.Cfg(S=1200, H=512, I=512, E=2, k=2, act=ob.ACT_GELU, dtype=ob.F16, drop=1, capacity_factor=0.9),
    # most experts empty, one row here and there
    "gelu_sparse_experts": ob.Cfg(S=40, H=256, I=256, E=32, k=1, act=ob.ACT_GELU, dtype=ob.BF16, norm_topk=0, drop=0),
    "relu_bias_capacity_drop": ob.Cfg(S=1100, H=512, I=256, E=2, k=2, act=ob.ACT_RELU, dtype=ob.BF16, drop=1,
                                      capacity_factor=0.7),
}


@pytest.mark.parametrize("name", sorted(LARGE_TILE))
def test_large_tile_and_queue_groups(moe, name):
    """The 256-row tile forced on small layers, in both FFN modes and with 1, 2 and 8 task queues: every run must
    reproduce the first bit for bit (the schedule only reorders independent tiles) and match the oracle."""
    cfg = LARGE_TILE[name]
    inp = ob.make_inputs(cfg, seed=5, with_bias="bias" in name)
    want = ob.forward(cfg, inp)
    first = None
    for groups in (1, 2, 8):
        opts = {"block_rows": 256, "queue_groups": groups}
        for mode in (FFN_TILED, FFN_PERSISTENT):
            got = run_layer(moe, cfg, inp, mode, opts)
            check_routing(got, want)
            eligible = cfg.H % 256 == 0 and cfg.I % (128 if cfg.act == ob.ACT_SWIGLU else 256) == 0
            assert got["plan"]["block_rows"] == (256 if eligible else 128)     # the cases cover both tiles
            if first is None:
                first = got["out"]
                assert max_rel_err(ob.to_f32(first, cfg.act_dtype), ob.to_f32(want["out"], cfg.act_dtype)) <= OUT_TOL[cfg.dtype]
            else:
                assert np.array_equal(got["out"], first), (groups, mode)
        # the queue loop that starts the next task under the end of the current one (same tiles, other timing)
        got = run_layer(moe, cfg, inp, FFN_PERSISTENT, dict(opts, queue_early=1))
        check_routing(got, want)
        assert np.array_equal(got["out"], first), ("early", groups)


@pytest.mark.parametrize("name", ["bf16_gelu_ragged", "bf16_swiglu_skew", "f32_swiglu_ragged", "fp8_many_rows_bias",
                                  "fp16_swiglu_skew_bias", "tf32_gelu_ragged", "capacity_one", "many_experts_bias",
                                  "all_experts_selected", "one_token"])
@pytest.mark.parametrize("combine", [1, 2], ids=["arrival_counters", "queue_tasks"])
def test_combine_inside_the_ffn_kernels_changes_no_bit(moe, name, combine):
    """Option combine = 1: a token is combined by the FFN workgroup that stores its last expert row; 2: by workgroups of
    the queue kernel that find no GEMM task left (the rest by a short launch behind it); 0: a launch of its own behind
    the FFN stage.  Same function, same rank order: the outputs must be identical in every bit, in both FFN modes,
    including the all-zero rows of tokens that lost every pair to the capacity limit, and over repeated calls on one
    handle (the counters are cleared by every call)."""
    import torch
    cfg = RAGGED[name]
    inp = ob.make_inputs(cfg, seed=3, with_bias="bias" in name)
    separate = run_layer(moe, cfg, inp, FFN_TILED, {"combine": 0})["out"]
    for mode in (FFN_TILED, FFN_PERSISTENT):
        layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, options={"combine": combine})
        dev = upload_inputs(cfg, inp)
        for call in range(3):
            out = torch.full((cfg.S, cfg.H), float("nan"), dtype=layer.act_dtype, device="cuda")   # nothing may be left unwritten
            layer.forward(dev["x"], dev, out=out)
            torch.cuda.synchronize()
            assert np.array_equal(from_device(out), separate), (mode, call)
        assert layer.stage_ms is not None
        layer.close()


@pytest.mark.parametrize("name", sorted(n for n, c in LARGE_TILE.items()
                                        if c.H % 256 == 0 and c.I % (128 if c.act == ob.ACT_SWIGLU else 256) == 0))
def test_half_height_tile(moe, name):
    """The 128 x 256 tile as the tile of the whole layer (option tile16 = 2) and as the tile of the short last row blocks
    only (3): every output element is accumulated by the same MFMA sequence over K as in the 256 x 256 tile, so all
    three must agree bit for bit, in both FFN modes, and match the oracle."""
    cfg = LARGE_TILE[name]
    inp = ob.make_inputs(cfg, seed=5, with_bias="bias" in name)
    want = ob.forward(cfg, inp)
    first = None
    for tile, rows in ((1, 256), (2, 128), (3, 256)):
        for mode in (FFN_TILED, FFN_PERSISTENT):
            got = run_layer(moe, cfg, inp, mode, {"tile16": tile})
            check_routing(got, want)
            assert got["plan"]["block_rows"] == rows
            if first is None:
                first = got["out"]
                assert max_rel_err(ob.to_f32(first, cfg.act_dtype), ob.to_f32(want["out"], cfg.act_dtype)) <= OUT_TOL[cfg.dtype]
            else:
                assert np.array_equal(got["out"], first), (tile, mode)


def test_two_handles_on_two_streams_from_two_threads(moe):
    """The boundary promises that handles are independent: two layers, each driven from its own host thread on its
    own (default-priority) stream, overlap freely and must reproduce what each computes alone."""
    import threading
    import torch
    cases = [RAGGED["bf16_swiglu_skew"], RAGGED["bf16_gelu_ragged"]]
    layers, devs, alone = [], [], []
    for cfg in cases:
        inp = ob.make_inputs(cfg, seed=9)
        layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT)
        dev = upload_inputs(cfg, inp)
        alone.append(layer.forward(dev["x"], dev).clone())
        layers.append(layer)
        devs.append(dev)
    torch.cuda.synchronize()
    results, errors = [None, None], []

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            outs = []
            with torch.cuda.stream(stream):
                for _ in range(20):
                    outs.append(layers[i].forward(devs[i]["x"], devs[i]).clone())
            stream.synchronize()
            layers[i].task_counts()
            results[i] = outs
        except Exception as e:      # surfaced in the main thread
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not errors, errors
    for i in range(2):
        assert results[i] is not None and all(torch.equal(o, alone[i]) for o in results[i])
        layers[i].close()


GRAPH_CASES = {
    "bf16": (None, {}),
    # an e4m3 layer on the widening plan (three more launches per call, the workspace copy rewritten by every replay)
    "e4m3_widened": (ob.Cfg(S=600, H=256, I=384, E=4, k=2, act=ob.ACT_SWIGLU, dtype=ob.FP8, gate_fn=ob.GATE_SIGMOID, drop=0),
                     {"fp8_widen": 1}),
    # an fp32 layer on the matrix-core tile, and a 16-bit one whose logits come from the matrix-core gate kernel
    "f32_tile": (ob.Cfg(S=500, H=256, I=256, E=2, k=1, act=ob.ACT_GELU, dtype=ob.F32, norm_topk=0, drop=0),
                 {"f32_tile": 1}),
    "f16_gate_mfma": (ob.Cfg(S=300, H=512, I=128, E=20, k=3, act=ob.ACT_RELU, dtype=ob.F16, drop=1, capacity_factor=1.0),
                      {"gate_mfma": 1}),
}


@pytest.mark.parametrize("mode", [FFN_TILED, FFN_PERSISTENT], ids=["tiled", "persistent"])
@pytest.mark.parametrize("case", sorted(GRAPH_CASES))
def test_forward_under_graph_capture(moe, mode, case):
    """moe_forward only enqueues kernels: it can be captured into a HIP graph.  The graph is replayed several times
    with eager work and synchronisations in between, on changing inputs, and every replay is checked against the
    eager result for the same input."""
    import torch
    cfg, options = GRAPH_CASES[case]
    cfg = cfg or RAGGED["bf16_swiglu_bias_dropless"]
    inp = ob.make_inputs(cfg, seed=13, with_bias=case == "bf16")
    layer = moe.MoELayer(product_config(cfg), ffn_mode=mode, options=options)
    dev = upload_inputs(cfg, inp)
    x = dev["x"].clone()
    out = torch.empty_like(x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer.forward(x, dev, out=out)            # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        layer.forward(x, dev, out=out)
    g = torch.Generator(device="cuda").manual_seed(3)
    for it in range(4):
        x.copy_(torch.randn(x.shape, device="cuda", generator=g).to(x.dtype))     # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = layer.forward(x, dev)
        torch.cuda.synchronize()
        assert torch.equal(got, want), it
    layer.task_counts()
    layer.close()
