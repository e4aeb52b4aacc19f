"""The BASELINE configurations at full size on the GPU.

The oracle cannot run a whole 5.8 TFLOP layer in test time, so: routing (integers) is compared in full, the
layer output on a stratified sample of tokens (each expert's first row, tail block, wavefront and row-block
boundaries, plus a few hundred random tokens), and the rest through properties that hold at any size (the two
independent FFN schedules agree bit for bit, fully dropped tokens are exactly zero, kept rows add up)."""
import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, from_device, max_rel_err, product_config, upload_inputs

pytestmark = pytest.mark.gpu
FFN_TILED, FFN_PERSISTENT = 1, 2
RANDOM_TOKENS = {"C2": 512, "C3": 256, "C4": 512, "C5": 64, "R0": 256, "X1": 128}   # C5: all of its tokens
MAX_STRATA_EXPERTS = 32
# Two more full-size layers beside the five measured configurations: the knob file the reference ships
# (aristos_config.json: fp32, 4 x 2048 tokens, one expert, ReLU -- the fp32 matrix-core tile), and the Mixtral shape
# with e4m3 weights (the plan that widens the weights to bf16 in the workspace).
FULL_SIZE = dict(ob.BASELINE)
FULL_SIZE["R0"] = ob.Cfg(S=8192, H=1024, I=4096, E=1, k=1, act=ob.ACT_RELU, dtype=ob.F32, norm_topk=0, drop=0)
FULL_SIZE["X1"] = ob.BASELINE["C3"].scaled(dtype=ob.FP8)


def stratified_tokens(cfg, want, block_rows, seed=7):
    """Tokens whose rows sit where a tile kernel is most likely to go wrong, plus a seeded random sample.

    Per expert (the 32 most loaded when there are more): the first packed row, the last row (the end of the partial
    tail block), the rows either side of the first 128-row wavefront boundary, either side of the first row-block
    boundary, and the first row of the tail block.  Returns (tokens, strata) with strata a list of
    (expert, slot, row block, what)."""
    cnt, off, tok = want["expert_count"], want["expert_offset"], want["token_indices"]
    experts = [int(e) for e in np.argsort(-cnt, kind="stable")[:MAX_STRATA_EXPERTS] if cnt[e] > 0]
    strata = []
    for e in sorted(experts):
        n = int(cnt[e])
        tail0 = (n - 1) // block_rows * block_rows
        picks = {0: "first", n - 1: "last row of the tail block", tail0: "first row of the tail block"}
        for b, what in ((128, "128-row wavefront boundary"), (block_rows, "row-block boundary")):
            if n > b:
                picks.setdefault(b - 1, "below the " + what)
                picks.setdefault(b, "above the " + what)
        for slot, what in sorted(picks.items()):
            strata.append((e, slot, slot // block_rows, what))
    chosen = [int(tok[off[e] + slot]) for e, slot, _, _ in strata]
    return chosen, strata, np.random.default_rng(seed)


@pytest.mark.parametrize("name", ["C2", "C3", "C4", "C5", "R0", "X1"])
def test_baseline_config_full_size(name):
    import torch
    import cuplayground_amd as moe
    assert torch.cuda.is_available()
    cfg = FULL_SIZE[name]
    print("config", name, cfg, flush=True)
    inp = ob.make_inputs(cfg, seed=42)
    want = ob.route(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT)
    dev = upload_inputs(cfg, inp)
    if name == "R0":
        assert layer.plan["block_rows"] == 128             # the matrix-core tile, not the 64-row vector one
    if name == "X1":
        assert layer.kernel_dtype == ob.BF16               # widened weights, bf16 kernels
    routing = layer.new_routing()
    out = layer.forward(dev["x"], dev, routing=routing)
    torch.cuda.synchronize()
    t0, t1 = layer.task_counts()
    got = {k: from_device(v) for k, v in routing.items()}
    for key in ("topk_idx", "slot", "expert_count", "expert_offset", "token_indices"):
        assert np.array_equal(got[key], want[key]), key
    assert np.abs(got["topk_w"] - want["topk_w"]).max() <= 2e-6
    kept = int(want["expert_count"].sum())
    assert kept == int((want["slot"] >= 0).sum())
    if not cfg.drop:
        assert kept == cfg.S * cfg.k
    assert t0 > 0 and t1 > 0

    # sampled output parity: stratified rows (tails, wavefront and row-block boundaries) + a seeded random sample,
    # always including a token with a dropped pair if there is one
    chosen, strata, rng = stratified_tokens(cfg, want, layer.plan["block_rows"])
    rand = rng.choice(cfg.S, size=min(RANDOM_TOKENS[name], cfg.S), replace=False)
    partly = np.nonzero((want["slot"] < 0).any(axis=1))[0]
    tokens = np.unique(np.concatenate([chosen, rand, partly[:4]])).astype(np.int32)
    tails = sum(1 for s_ in strata if "tail" in s_[3])
    print(name, "block rows", layer.plan["block_rows"], "strata", len(strata), "over experts",
          sorted({s_[0] for s_ in strata}), "tail rows", tails, "tokens checked", tokens.size, flush=True)
    for s_ in strata[:12]:
        print("   stratum expert %d slot %d row block %d: %s" % s_, flush=True)
    ref = ob.to_f32(ob.forward_tokens(cfg, inp, want["topk_idx"], want["topk_w"], want["slot"], tokens), cfg.act_dtype)
    o = out.float().cpu().numpy()
    err = max_rel_err(o[tokens], ref)
    print(name, "sampled max rel err", err, flush=True)
    assert err <= OUT_TOL[cfg.dtype], err

    dead = (want["slot"] < 0).all(axis=1)
    assert (o[dead] == 0).all()
    assert np.isfinite(o).all()

    # the two-launch schedule shares no queue state with the persistent one and must agree bit for bit
    layer.set_ffn_mode(FFN_TILED)
    out2 = layer.forward(dev["x"], dev)
    assert torch.equal(out, out2)
    # and so must the queue loop with the early start of the next task (an opt-in schedule of the 256-row tile)
    layer.close()
    early = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT, options={"queue_early": 1})
    out3 = early.forward(dev["x"], dev)
    torch.cuda.synchronize()
    early.task_counts()
    assert torch.equal(out, out3)
    early.close()


@pytest.mark.parametrize("S,H,I,k,rows", [(100000, 256, 8192, 2, 256), (140000, 256, 8192, 2, 128), (300000, 4096, 256, 1, 256)],
                         ids=["h_3GiB_large_tile", "h_4.6GiB_small_tile", "x_2.4GiB_large_tile"])
def test_operands_beyond_2_and_4_gib(S, H, I, k, rows):
    """Byte offsets that need bit 31 (the 256-row tile addresses its operands through 32-bit unsigned buffer offsets:
    the intermediate buffer in the first case, the gathered token rows in the third) and that exceed 32 bits (the
    layer then has to fall back to the 128-row tile, which uses 64-bit addresses).  With k = 2 every token goes to
    both experts, so the second expert's rows sit in the upper half of the intermediate buffer."""
    import torch
    import cuplayground_amd as moe
    cfg = ob.Cfg(S=S, H=H, I=I, E=2, k=k, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=0, norm_topk=0)
    biggest = max(S * H * 2, S * k * I * 2)
    assert biggest > 2 ** 31 and (biggest >= 2 ** 32) == (rows == 128)
    inp = ob.make_inputs(cfg, seed=4)
    want = ob.route(cfg, inp)
    layer = moe.MoELayer(product_config(cfg), ffn_mode=FFN_PERSISTENT)
    assert layer.plan["block_rows"] == rows
    dev = upload_inputs(cfg, inp)
    routing = layer.new_routing()
    out = layer.forward(dev["x"], dev, routing=routing)
    torch.cuda.synchronize()
    layer.task_counts()
    got = {k: from_device(v) for k, v in routing.items()}
    for key in ("topk_idx", "slot", "expert_count", "expert_offset"):
        assert np.array_equal(got[key], want[key]), key
    # tokens whose rows lie at the very end of each expert's range, plus a random handful
    rng = np.random.default_rng(1)
    tokens = np.concatenate([[0, 1, S // 2, S - 2, S - 1], rng.choice(S, size=27, replace=False)]).astype(np.int32)
    ref = ob.to_f32(ob.forward_tokens(cfg, inp, want["topk_idx"], want["topk_w"], want["slot"], tokens), cfg.act_dtype)
    o = out[torch.from_numpy(tokens.astype(np.int64)).cuda()].float().cpu().numpy()
    err = max_rel_err(o, ref)
    print("S", S, "block rows", rows, "sampled max rel err", err, flush=True)
    assert err <= OUT_TOL[cfg.dtype], err
    layer.set_ffn_mode(FFN_TILED)
    out2 = layer.forward(dev["x"], dev)
    assert torch.equal(out, out2)
    layer.close()
