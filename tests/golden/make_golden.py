"""Writes the golden fixtures of this directory from the CPU oracle.

Run from the repository root:  python tests/golden/make_golden.py
  c1_layer.npz        the tiny fp32 configuration in full: routing result and layer output
  routing_digests.json  per BASELINE configuration: expert_count and SHA-256 of topk_idx / slot, full size
Inputs are not stored: they are regenerated from (seed, tensor id) by the oracle's counter-based generator.
Before writing, the C1 output is cross-checked against a float64 torch-CPU evaluation of the same layer.
"""
import hashlib
import json
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding as ob  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
SEED = 42


def torch_c1(cfg, inp, r):
    x = torch.from_numpy(inp["x"]).double()
    logits = x @ torch.from_numpy(inp["gate_w"]).double().T
    p = torch.softmax(logits, dim=1)
    top = logits.argmax(dim=1)
    out = torch.zeros(cfg.S, cfg.H, dtype=torch.float64)
    for t in range(cfg.S):
        if r["slot"][t, 0] < 0:
            continue
        e = int(top[t])
        h = torch.nn.functional.gelu(torch.from_numpy(inp["w_up"][e]).double() @ x[t])
        out[t] = p[t, e] * (torch.from_numpy(inp["w_down"][e]).double() @ h)
    return top.numpy(), out.numpy()


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    cfg = ob.BASELINE["C1"]
    inp = ob.make_inputs(cfg, SEED)
    r = ob.forward(cfg, inp)
    top, want = torch_c1(cfg, inp, r)
    assert np.array_equal(top, r["topk_idx"][:, 0])
    assert np.abs(r["out"] - want).max() <= 1e-5 * np.abs(want).max()
    np.savez_compressed(os.path.join(HERE, "c1_layer.npz"), out=r["out"], topk_idx=r["topk_idx"], topk_w=r["topk_w"],
                        slot=r["slot"], expert_count=r["expert_count"], expert_offset=r["expert_offset"],
                        token_indices=r["token_indices"])
    digests = {}
    for name, c in ob.BASELINE.items():
        rr = ob.route(c, ob.make_inputs(c, SEED, router_only=True))
        l = np.sort(rr["logits"], axis=1)[:, ::-1]
        digests[name] = dict(
            seed=SEED, S=c.S, E=c.E, k=c.k, capacity=c.capacity if c.drop else None,
            expert_count=[int(v) for v in rr["expert_count"]],
            dropped_pairs=int((rr["slot"] < 0).sum()),
            min_topk_margin=float((l[:, c.k - 1] - l[:, c.k]).min()) if c.E > c.k else None,
            topk_idx_sha256=digest(rr["topk_idx"]), slot_sha256=digest(rr["slot"]),
            logits_sha256=digest(rr["logits"]))
        print(name, digests[name]["dropped_pairs"], digests[name]["min_topk_margin"], flush=True)
    with open(os.path.join(HERE, "routing_digests.json"), "w") as f:
        json.dump(digests, f, indent=1)


if __name__ == "__main__":
    main()
