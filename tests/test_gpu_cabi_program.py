"""The C ABI called from a C++ program (tests/cabi/run_layer.cpp, built by __graft_entry__.build()), no Python in
the process that runs the layer; its outputs are checked against the CPU oracle."""
import os
import subprocess

import numpy as np
import pytest

from oracle import binding as ob
from helpers import OUT_TOL, as_f32, max_rel_err, product_config

pytestmark = pytest.mark.gpu
PROGRAM = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cabi", "run_layer")

CASES = {
    "bf16_swiglu": ob.Cfg(S=384, H=256, I=384, E=8, k=2, act=ob.ACT_SWIGLU, dtype=ob.BF16, drop=1, capacity_factor=1.0),
    "f32_gelu": ob.Cfg(S=128, H=128, I=256, E=4, k=1, act=ob.ACT_GELU, dtype=ob.F32, norm_topk=0, drop=0),
    # the knob values of the reference's own aristos_config.json at one of its four micro-batches: fp32, one expert,
    # ReLU, H 1024, I 4096 -- the plan that runs the fp32 matrix-core tile
    "f32_reference_knobs": ob.Cfg(S=2048, H=1024, I=4096, E=1, k=1, act=ob.ACT_RELU, dtype=ob.F32, norm_topk=0, drop=0,
                                  capacity_factor=1.0),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_cpp_caller_matches_oracle(tmp_path, name):
    assert os.path.exists(PROGRAM), "tests/cabi/run_layer is missing: run __graft_entry__.build() first"
    cfg = CASES[name]
    inp = ob.make_inputs(cfg, seed=31)
    want = ob.forward(cfg, inp)
    (tmp_path / "config.json").write_text(product_config(cfg).to_json())
    for key in ("x", "gate_w", "w_up", "w_gate", "w_down"):
        if inp.get(key) is not None:
            np.ascontiguousarray(inp[key]).tofile(tmp_path / (key + ".bin"))
    run = subprocess.run([PROGRAM, str(tmp_path / "config.json"), str(tmp_path)], capture_output=True, text=True,
                         timeout=100)
    assert run.returncode == 0, run.stderr + run.stdout
    assert run.stdout.startswith("ok tokens=%d " % cfg.S)
    S, k = cfg.S, cfg.k
    assert np.array_equal(np.fromfile(tmp_path / "topk_idx.bin", np.int32).reshape(S, k), want["topk_idx"])
    assert np.array_equal(np.fromfile(tmp_path / "slot.bin", np.int32).reshape(S, k), want["slot"])
    assert np.array_equal(np.fromfile(tmp_path / "expert_count.bin", np.int32), want["expert_count"])
    raw = np.fromfile(tmp_path / "out.bin", np.float32 if cfg.dtype == ob.F32 else np.uint16).reshape(S, cfg.H)
    assert max_rel_err(as_f32(raw, cfg.dtype), as_f32(want["out"], cfg.dtype)) <= OUT_TOL[cfg.dtype]


def test_cpp_caller_reports_a_bad_config(tmp_path):
    assert os.path.exists(PROGRAM), "tests/cabi/run_layer is missing: run __graft_entry__.build() first"
    (tmp_path / "config.json").write_text('{"hidden_size": 100}')
    run = subprocess.run([PROGRAM, str(tmp_path / "config.json"), str(tmp_path)], capture_output=True, text=True,
                         timeout=100)
    assert run.returncode == 3 and "config:" in run.stderr
