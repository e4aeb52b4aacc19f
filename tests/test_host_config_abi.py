"""Host-side checks that need no GPU: the C-ABI library loads, exports what the header declares, and its
config loader implements the reference schema (aristos_config.schema.json) plus the documented relaxations."""
import ctypes as C
import json
import os
import re

import pytest

import cuplayground_amd as moe
from cuplayground_amd import api

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REFERENCE_JSON = {  # the values of the reference's own aristos_config.json:1-13
    "capacity_factor": 1, "drop_tokens": 0, "expert_top_k": 1, "is_training": 0, "hidden_act": 0, "hidden_size": 1024,
    "intermediate_size": 4096, "micro_batch": 4, "num_experts": 1, "sequence_len": 2048, "torch_dtype": 0}


def test_library_exports_every_declared_symbol():
    L = moe.load_library()
    header = open(os.path.join(ROOT, "include", "moe355.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", header))
    assert declared == set(api.EXPORTS)
    for name in declared:
        assert hasattr(L, name), name
    assert L.moe_version() == 1
    assert L.moe_status_string(0) == b"ok" and L.moe_status_string(3).startswith(b"workspace")


def test_reference_config_file_loads_unchanged(tmp_path):
    p = tmp_path / "aristos_config.json"
    p.write_text(json.dumps(REFERENCE_JSON, indent=2))
    cfg = moe.MoEConfig.from_json(str(p))
    for k, v in REFERENCE_JSON.items():
        assert getattr(cfg, k) == v
    assert cfg.gate_fn == 0 and cfg.norm_topk_prob == 0
    assert cfg.tokens == 4 * 2048
    assert moe.MoEConfig.from_json(json.dumps(REFERENCE_JSON)) == cfg


def test_defaults_are_the_reference_file():
    c = api._CConfig()
    assert moe.load_library().moe_config_default(C.byref(c)) == 0
    assert moe.MoEConfig._from_c(c) == moe.MoEConfig(**REFERENCE_JSON)


@pytest.mark.parametrize("key", ["hidden_act", "hidden_size", "intermediate_size", "expert_top_k", "capacity_factor",
                                 "drop_tokens", "num_experts", "sequence_len", "micro_batch", "torch_dtype"])
def test_required_keys(key):   # aristos_config.schema.json:60-71
    d = dict(REFERENCE_JSON); del d[key]
    with pytest.raises(moe.MoEError) as e:
        moe.MoEConfig.from_json(json.dumps(d))
    assert e.value.status == 1 and key in str(e.value)


def test_is_training_is_optional_and_extra_keys_are_ignored():
    d = dict(REFERENCE_JSON); del d["is_training"]
    d["$schema"] = "x"; d["note"] = {"nested": [1, 2, {"a": "}"}]}
    assert moe.MoEConfig.from_json(json.dumps(d)).is_training == 0


@pytest.mark.parametrize("patch", [
    {"capacity_factor": 0}, {"capacity_factor": -1.5}, {"drop_tokens": 2}, {"expert_top_k": 0}, {"expert_top_k": 1.5},
    {"is_training": 3}, {"hidden_act": 3}, {"hidden_act": -1}, {"hidden_size": 1000}, {"hidden_size": 0},
    {"intermediate_size": 4100}, {"micro_batch": 0}, {"num_experts": 0}, {"sequence_len": 0}, {"torch_dtype": 5},
    {"gate_fn": 2}, {"norm_topk_prob": 2}, {"expert_top_k": 2, "num_experts": 1}, {"hidden_size": 64.5},
])
def test_domain_violations_are_rejected(patch):
    d = dict(REFERENCE_JSON); d.update(patch)
    with pytest.raises(moe.MoEError) as e:
        moe.MoEConfig.from_json(json.dumps(d))
    assert e.value.status == 1


@pytest.mark.parametrize("text", ["", "[]", "{", '{"a" 1}', '{"hidden_size": }', '{"hidden_size": 64,}', "{} x"])
def test_malformed_json(text):
    with pytest.raises(moe.MoEError) as e:
        moe.MoEConfig.from_json(text)
    assert e.value.status == 1


def test_extensions_and_relaxations():
    d = dict(REFERENCE_JSON)
    d.update(capacity_factor=1.25, hidden_act=2, torch_dtype=4, sequence_len=64, micro_batch=1, num_experts=256,
             expert_top_k=8, gate_fn=1, hidden_size=7168, intermediate_size=2048)
    cfg = moe.MoEConfig.from_json(json.dumps(d))
    assert cfg.capacity_factor == 1.25 and cfg.tokens == 64 and cfg.norm_topk_prob == 1   # default on for k > 1
    d["norm_topk_prob"] = 0
    assert moe.MoEConfig.from_json(json.dumps(d)).norm_topk_prob == 0
    assert moe.MoEConfig.from_json(moe.MoEConfig(**REFERENCE_JSON).to_json()) == moe.MoEConfig(**REFERENCE_JSON)


def test_capacity_matches_oracle(oracle):
    for name, c in oracle.BASELINE.items():
        pc = moe.MoEConfig(capacity_factor=c.capacity_factor, expert_top_k=c.k, num_experts=c.E, micro_batch=1,
                           sequence_len=c.S)
        assert pc.capacity == c.capacity, name


def test_workspace_and_unsupported_shapes():
    base = dict(capacity_factor=1.0, drop_tokens=1, expert_top_k=2, hidden_act=1, hidden_size=256, intermediate_size=512,
                micro_batch=1, num_experts=8, sequence_len=128, torch_dtype=2)
    small = moe.MoEConfig(**base).workspace_bytes()
    big = moe.MoEConfig(**{**base, "sequence_len": 256}).workspace_bytes()
    assert 0 < small < big and small % 256 == 0
    # at least the two intermediates: h [A,I] and y [A,H] in bf16
    assert small >= 128 * 2 * (512 + 256) * 2
    # every dtype of the reference schema has a kernel: tf32 is stored and computed as fp32 (twice the bytes of bf16)
    assert moe.MoEConfig(**{**base, "torch_dtype": 3}).workspace_bytes() == small
    assert moe.MoEConfig(**{**base, "torch_dtype": 1}).workspace_bytes() == moe.MoEConfig(**{**base, "torch_dtype": 0}).workspace_bytes() > small
    # e4m3 layers take every activation; their sizes are multiples of the 128 x 128 scale block
    assert moe.MoEConfig(**{**base, "torch_dtype": 4}).workspace_bytes() > 0
    with pytest.raises(moe.MoEError) as e:
        moe.MoEConfig(**{**base, "torch_dtype": 4, "intermediate_size": 192}).workspace_bytes()
    assert e.value.status == 2
    for patch in ({"num_experts": 1024}, {"expert_top_k": 17, "num_experts": 64}, {"hidden_size": 32768}):
        with pytest.raises(moe.MoEError) as e:
            moe.MoEConfig(**{**base, **patch}).workspace_bytes()
        assert e.value.status == 2
    with pytest.raises(moe.MoEError) as e:
        moe.MoEConfig(**{**base, "hidden_size": 100}).workspace_bytes()
    assert e.value.status == 1


def test_options_default_env_and_domains(monkeypatch):
    """moe_options: defaults are all AUTO; the environment is read by moe_options_from_env only (and by the entry points
    that take no options), values outside a field's domain are ignored there and refused by the *_with_options entries;
    the workspace follows the options, not the environment, when options are given."""
    import ctypes as C
    from cuplayground_amd import api
    L = moe.load_library()
    o = api.make_options()
    assert all(getattr(o, n) == api.OPT_AUTO for n in api.OPTION_FIELDS) and all(v == api.OPT_AUTO for v in o.reserved)
    for name in api.OPTION_FIELDS:
        monkeypatch.delenv("MOE355_" + name.upper(), raising=False)
    monkeypatch.setenv("MOE355_FP8_WIDEN", "1")
    monkeypatch.setenv("MOE355_QUEUE_GROUPS", "3")       # not a power of two: ignored
    monkeypatch.setenv("MOE355_TILE16", "x")             # not a number: ignored
    monkeypatch.setenv("MOE355_COMBINE", "2")
    e = api.make_options(from_env=True)
    assert (e.fp8_widen, e.queue_groups, e.tile16, e.combine) == (1, api.OPT_AUTO, api.OPT_AUTO, 2)
    cfg = moe.MoEConfig(capacity_factor=1.0, drop_tokens=0, expert_top_k=2, hidden_act=2, hidden_size=256,
                        intermediate_size=256, micro_batch=1, num_experts=4, sequence_len=256, torch_dtype=4)
    c = cfg.to_c()

    def ws(opts):
        n = C.c_size_t(0)
        rc = L.moe_workspace_bytes_with_options(C.byref(c), C.byref(api.make_options(opts)), C.byref(n))
        return rc, n.value

    rc0, plain = ws({"fp8_widen": 0})
    rc1, wide = ws({"fp8_widen": 1})
    assert rc0 == 0 and rc1 == 0 and wide - plain >= 3 * 4 * 256 * 256 * 2    # the bf16 copies of three weight matrices
    assert cfg.workspace_bytes() == wide                   # no options argument: MOE355_FP8_WIDEN=1 from the environment
    monkeypatch.delenv("MOE355_FP8_WIDEN")
    assert cfg.workspace_bytes() == ws({})[1] == plain     # 128 rows per expert: below the widening threshold
    for bad in ({"tile16": 4}, {"queue_groups": 3}, {"block_rows": 200}, {"combine": 3}, {"tail_round": 2}, {"tail_split": 3}, {"tail_split": 0},
                {"blocks_per_cu": 0}, {"fp8_tile": -2}):
        assert ws(bad)[0] == 4, bad
    r = api.make_options()
    r.reserved[3] = 0
    n = C.c_size_t(0)
    assert L.moe_workspace_bytes_with_options(C.byref(c), C.byref(r), C.byref(n)) == 4
    with pytest.raises(KeyError):
        api.make_options({"no_such_option": 1})


def test_null_arguments_are_errors_not_crashes():
    L = moe.load_library()
    assert L.moe_config_default(None) == 4
    assert L.moe_workspace_bytes(None, None) == 4
    assert L.moe_create(None, None) == 4
    assert L.moe_create_with_options(None, None, None) == 4
    assert L.moe_options_default(None) == 4 and L.moe_options_from_env(None) == 4
    assert L.moe_get_options(None, None) == 4 and L.moe_get_workspace_bytes(None, None) == 4
    assert L.moe_get_stall(None, None) == 4
    assert L.moe_prepared_bytes(None, None) == 4 and L.moe_prepare_weights(None, None, None, 0, None) == 4
    assert L.moe_destroy(None) == 0
    assert L.moe_forward(None, None, None, None, None, None, 0, None) == 4
    assert L.moe_gemm_bias_act(None, None, None, None, 1, 1, 1, 0, 0, None) == 4


def test_torch_operator_has_no_cpu_path():
    """The operator is declared for CUDA (and meta) only: CPU tensors must be refused by the dispatcher."""
    import torch
    import cuplayground_amd.torch_op  # noqa: F401  (registers torch.ops.moe355.forward)
    x = torch.zeros(128, 64)
    w = torch.zeros(2, 64)
    e = torch.zeros(2, 64, 64)
    cfg = '{"hidden_size": 64, "intermediate_size": 64, "num_experts": 2, "sequence_len": 128, "micro_batch": 1}'
    with pytest.raises((NotImplementedError, RuntimeError)):
        torch.ops.moe355.forward(x, w, e, None, e, cfg)
    m = torch.ops.moe355.forward(x.to("meta"), w.to("meta"), e.to("meta"), None, e.to("meta"), cfg)
    assert m.shape == x.shape
