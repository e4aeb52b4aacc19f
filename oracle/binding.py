"""ctypes/numpy wrapper around liboracle.so -- TEST INFRASTRUCTURE ONLY (see moe_oracle.h).

bf16 tensors travel as numpy uint16 arrays holding the raw bit patterns, e4m3 tensors as uint8.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess
from dataclasses import dataclass, replace

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

F32, TF32, BF16, F16, FP8 = 0, 1, 2, 3, 4
ACT_RELU, ACT_GELU, ACT_SWIGLU, ACT_NONE = 0, 1, 2, 3
GATE_SOFTMAX, GATE_SIGMOID = 0, 1

# tensor ids for the seeded generator: element i of tensor `stream` is a pure function of (seed, stream, i)
STREAM = dict(x=1, gate_w=2, gate_bias=3, w_up=4, w_gate=5, w_down=6, b_up=7, b_gate=8, b_down=9)


def build(force: bool = False) -> str:
    """Compile liboracle.so with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH) or any(
        os.path.getmtime(os.path.join(_HERE, f)) > os.path.getmtime(_LIB_PATH)
        for f in ("moe_oracle.c", "moe_oracle.h", "Makefile")
    ):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True)
    return _LIB_PATH


class _Cfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("S", "H", "I", "E", "k", "act", "dtype", "gate_fn", "norm_topk", "drop")] + [
        ("capacity", C.c_int64)
    ]


class _Weights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "gate_w", "gate_bias", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "s_up", "s_gate", "s_down")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        vp, i32, i64, u64, f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_uint64, C.c_float
        L.orc_philox4x32_10.argtypes = [vp, vp, vp]
        L.orc_fill_normal.argtypes = [vp, i64, u64, u64, f32, f32]
        L.orc_fill_uniform.argtypes = [vp, i64, u64, u64]
        L.orc_f32_to_bf16.argtypes = [f32]; L.orc_f32_to_bf16.restype = C.c_uint16
        L.orc_bf16_to_f32.argtypes = [C.c_uint16]; L.orc_bf16_to_f32.restype = f32
        L.orc_f32_to_e4m3.argtypes = [f32]; L.orc_f32_to_e4m3.restype = C.c_uint8
        L.orc_e4m3_to_f32.argtypes = [C.c_uint8]; L.orc_e4m3_to_f32.restype = f32
        L.orc_round_bf16.argtypes = [vp, vp, i64]
        L.orc_widen_bf16.argtypes = [vp, vp, i64]
        L.orc_round_f16.argtypes = [vp, vp, i64]
        L.orc_widen_f16.argtypes = [vp, vp, i64]
        L.orc_f32_to_f16.argtypes = [f32]; L.orc_f32_to_f16.restype = C.c_uint16
        L.orc_f16_to_f32.argtypes = [C.c_uint16]; L.orc_f16_to_f32.restype = f32
        L.orc_quant_block128.argtypes = [vp, i64, i64, vp, vp]
        L.orc_dequant_block128.argtypes = [vp, vp, i64, i64, vp]
        L.orc_quant_rows128.argtypes = [vp, i64, i64, vp, vp]
        L.orc_dequant_rows128.argtypes = [vp, vp, i64, i64, vp]
        L.orc_capacity.argtypes = [C.c_double, i64, i64, i64, C.POINTER(i64)]
        L.orc_gate_logits.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
        L.orc_topk.argtypes = [vp, i32, i32, i32, i32, i32, vp, vp]
        L.orc_router_stats.argtypes = [vp, vp, i32, i32, i32, i32, vp, vp, vp]
        L.orc_route.argtypes = [vp, i32, i32, i32, i32, i64, vp, vp, vp, vp, vp]
        L.orc_gemm_bias_act.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32]
        L.orc_expert_gemm.argtypes = [vp, vp, vp, vp, vp, i32, i64, i64, i32, i32, vp]
        L.orc_expert_wgrad.argtypes = [vp, vp, vp, vp, i32, i64, i64, i32, vp]
        L.orc_act_backward.argtypes = [vp, vp, vp, i64, i64, i32, i32, vp, vp]
        L.orc_bias_grad.argtypes = [vp, vp, vp, i32, i64, i32, vp]
        L.orc_combine_backward.argtypes = [vp, vp, vp, vp, i32, i32, i32, i32, vp, vp]
        L.orc_ffn_rows.argtypes = [C.POINTER(_Cfg), vp, C.POINTER(_Weights), vp, vp, i64, vp]
        L.orc_combine.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp]
        L.orc_forward.argtypes = [C.POINTER(_Cfg), vp, C.POINTER(_Weights), vp, vp, vp, vp, vp, vp, vp]
        L.orc_forward_tokens.argtypes = [C.POINTER(_Cfg), vp, C.POINTER(_Weights), vp, vp, vp, vp, i64, vp]
        L.orc_num_threads.restype = C.c_int
        for fn in ("orc_philox4x32_10", "orc_fill_normal", "orc_fill_uniform", "orc_round_bf16", "orc_widen_bf16",
                   "orc_round_f16", "orc_widen_f16",
                   "orc_quant_block128", "orc_dequant_block128", "orc_quant_rows128", "orc_dequant_rows128", "orc_gate_logits", "orc_topk", "orc_route",
                   "orc_gemm_bias_act", "orc_expert_gemm", "orc_expert_wgrad", "orc_act_backward", "orc_bias_grad",
                   "orc_combine_backward", "orc_ffn_rows", "orc_combine", "orc_forward", "orc_forward_tokens"):
            getattr(L, fn).restype = None
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


# ---------------------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class Cfg:
    """One MoE layer shape.  Field meanings follow aristos_config.schema.json plus this build's extensions."""
    S: int
    H: int
    I: int
    E: int
    k: int
    act: int = ACT_GELU
    dtype: int = BF16
    gate_fn: int = GATE_SOFTMAX
    norm_topk: int = 1
    drop: int = 1
    capacity_factor: float = 1.0
    zipf_bias: bool = False   # C4: per-expert logit bias log(p_e), p_e ~ rank^-1.1

    @property
    def capacity(self) -> int:
        out = C.c_int64(0)
        rc = lib().orc_capacity(float(self.capacity_factor), self.S, self.k, self.E, C.byref(out))
        if rc:
            raise ValueError("bad capacity arguments")
        return out.value

    @property
    def act_dtype(self) -> int:
        """Storage type of activations: the layer's own, except fp32 for tf32 layers and bf16 for e4m3 layers."""
        if self.dtype in (F32, TF32):
            return F32
        return F16 if self.dtype == F16 else BF16

    def c_struct(self) -> _Cfg:
        return _Cfg(self.S, self.H, self.I, self.E, self.k, self.act, self.dtype, self.gate_fn, self.norm_topk,
                    self.drop, self.capacity)

    def scaled(self, **kw) -> "Cfg":
        return replace(self, **kw)


# The five BASELINE configurations.
BASELINE = {
    "C1": Cfg(S=128, H=256, I=512, E=8, k=1, act=ACT_GELU, dtype=F32, norm_topk=0, drop=1, capacity_factor=1.0),
    "C2": Cfg(S=4096, H=2048, I=2048, E=16, k=2, act=ACT_GELU, dtype=BF16, norm_topk=1, drop=1, capacity_factor=1.25),
    "C3": Cfg(S=8192, H=4096, I=14336, E=8, k=2, act=ACT_SWIGLU, dtype=BF16, norm_topk=1, drop=0, capacity_factor=2.0),
    "C4": Cfg(S=16384, H=2048, I=1408, E=64, k=6, act=ACT_SWIGLU, dtype=BF16, norm_topk=1, drop=1,
              capacity_factor=1.0, zipf_bias=True),
    "C5": Cfg(S=64, H=7168, I=2048, E=256, k=8, act=ACT_SWIGLU, dtype=FP8, gate_fn=GATE_SIGMOID, norm_topk=1,
              drop=0, capacity_factor=1.0),
}


# ---------------------------------------------------------------------------------------------------------
def philox(ctr, key):
    c = _c(ctr, np.uint32); k = _c(key, np.uint32); o = np.zeros(4, np.uint32)
    lib().orc_philox4x32_10(_p(c), _p(k), _p(o))
    return o


def normal(n, seed, stream, mean=0.0, std=1.0):
    a = np.empty(int(n), np.float32)
    lib().orc_fill_normal(_p(a), a.size, seed, stream, mean, std)
    return a


def uniform(n, seed, stream):
    a = np.empty(int(n), np.float32)
    lib().orc_fill_uniform(_p(a), a.size, seed, stream)
    return a


def f32_to_bf16(a):
    a = _c(a, np.float32); o = np.empty(a.shape, np.uint16)
    lib().orc_round_bf16(_p(a), _p(o), a.size)
    return o


def bf16_to_f32(a):
    a = _c(a, np.uint16); o = np.empty(a.shape, np.float32)
    lib().orc_widen_bf16(_p(a), _p(o), a.size)
    return o


def f32_to_f16(a):
    a = _c(a, np.float32); o = np.empty(a.shape, np.uint16)
    lib().orc_round_f16(_p(a), _p(o), a.size)
    return o


def f16_to_f32(a):
    a = _c(a, np.uint16); o = np.empty(a.shape, np.float32)
    lib().orc_widen_f16(_p(a), _p(o), a.size)
    return o


def to_f32(a, dtype):
    if dtype in (F32, TF32):
        return np.asarray(a, np.float32)
    return f16_to_f32(a) if dtype == F16 else bf16_to_f32(a)


def from_f32(a, dtype):
    """fp32 values rounded to an activation storage type (16-bit types as uint16 bit patterns)."""
    if dtype in (F32, TF32):
        return np.ascontiguousarray(a, np.float32)
    return f32_to_f16(a) if dtype == F16 else f32_to_bf16(a)


def quant_block128(w):
    """w: float32 [..., N, K] -> (uint8 same shape, float32 [..., ceil(N/128), ceil(K/128)])."""
    w = _c(w, np.float32)
    lead = w.shape[:-2]; N, K = w.shape[-2:]
    q = np.empty(w.shape, np.uint8)
    s = np.empty(lead + ((N + 127) // 128, (K + 127) // 128), np.float32)
    wf = w.reshape(-1, N, K); qf = q.reshape(-1, N, K); sf = s.reshape(-1, s.shape[-2], s.shape[-1])
    for i in range(wf.shape[0]):
        lib().orc_quant_block128(_p(wf[i]), N, K, _p(qf[i]), _p(sf[i]))
    return q, s


def dequant_block128(q, s):
    q = _c(q, np.uint8); s = _c(s, np.float32)
    N, K = q.shape[-2:]
    w = np.empty(q.shape, np.float32)
    qf = q.reshape(-1, N, K); wf = w.reshape(-1, N, K); sf = s.reshape(-1, s.shape[-2], s.shape[-1])
    for i in range(qf.shape[0]):
        lib().orc_dequant_block128(_p(qf[i]), _p(sf[i]), N, K, _p(wf[i]))
    return w


def quant_rows128(x):
    """x: float32 [R, K] -> (uint8 [R, K], float32 [R, ceil(K/128)]): e4m3 codes with one scale per row and 128 columns."""
    x = _c(x, np.float32)
    R, K = x.shape
    q = np.empty((R, K), np.uint8)
    s = np.empty((R, (K + 127) // 128), np.float32)
    lib().orc_quant_rows128(_p(x), R, K, _p(q), _p(s))
    return q, s


def dequant_rows128(q, s):
    q = _c(q, np.uint8); s = _c(s, np.float32)
    R, K = q.shape
    x = np.empty((R, K), np.float32)
    lib().orc_dequant_rows128(_p(q), _p(s), R, K, _p(x))
    return x


def zipf_gate_bias(E, seed, s=1.1):
    """log(p_e) with p_e proportional to rank_e^-s; the rank permutation is argsort of seeded uniforms."""
    u = uniform(E, seed, STREAM["gate_bias"])
    rank = np.empty(E, np.int64)
    rank[np.argsort(u, kind="stable")] = np.arange(1, E + 1)
    p = rank.astype(np.float64) ** (-s)
    p /= p.sum()
    return np.log(p).astype(np.float32)


def make_inputs(cfg: Cfg, seed: int = 42, with_bias: bool = False, router_only: bool = False) -> dict:
    """Seeded synthetic operands, already rounded to their storage types: tokens N(0,1), weights N(0,0.02).
    router_only skips the expert weights (enough for gate / top-k / slot checks at full size)."""
    S, H, I, E = cfg.S, cfg.H, cfg.I, cfg.E
    act = lambda a: from_f32(a, cfg.act_dtype)
    inp = {"x": act(normal(S * H, seed, STREAM["x"]).reshape(S, H)),
           "gate_w": act(normal(E * H, seed, STREAM["gate_w"], 0.0, 0.02).reshape(E, H)),
           "gate_bias": zipf_gate_bias(E, seed) if cfg.zipf_bias else None}
    names = ["w_up", "w_down"] + (["w_gate"] if cfg.act == ACT_SWIGLU else [])
    if router_only:
        return inp
    for n in names:
        shape = (E, H, I) if n == "w_down" else (E, I, H)
        w = normal(E * H * I, seed, STREAM[n], 0.0, 0.02).reshape(shape)
        if cfg.dtype in (F32, TF32):
            inp[n] = w
        elif cfg.dtype in (BF16, F16):
            inp[n] = from_f32(w, cfg.dtype)
        else:
            inp[n], inp["s_" + n[2:]] = quant_block128(w)
        del w
    if with_bias:
        inp["b_up"] = act(normal(E * I, seed, STREAM["b_up"], 0.0, 0.02).reshape(E, I))
        inp["b_down"] = act(normal(E * H, seed, STREAM["b_down"], 0.0, 0.02).reshape(E, H))
        if cfg.act == ACT_SWIGLU:
            inp["b_gate"] = act(normal(E * I, seed, STREAM["b_gate"], 0.0, 0.02).reshape(E, I))
    return inp


def _weights(inp) -> _Weights:
    w = _Weights()
    for n, _ in _Weights._fields_:
        a = inp.get(n)
        setattr(w, n, None if a is None else a.ctypes.data)
    return w


def gate_logits(x, gate_w, gate_bias, act_dtype):
    S, H = x.shape; E = gate_w.shape[0]
    out = np.empty((S, E), np.float32)
    gb = None if gate_bias is None else _c(gate_bias, np.float32)
    lib().orc_gate_logits(_p(np.ascontiguousarray(x)), _p(np.ascontiguousarray(gate_w)), _p(gb), S, H, E, act_dtype,
                          _p(out))
    return out


def topk(logits, k, gate_fn, norm_topk):
    logits = _c(logits, np.float32)
    S, E = logits.shape
    idx = np.empty((S, k), np.int32); w = np.empty((S, k), np.float32)
    lib().orc_topk(_p(logits), S, E, k, gate_fn, norm_topk, _p(idx), _p(w))
    return idx, w


def router_stats(logits, topk_idx, gate_fn):
    logits = _c(logits, np.float32); topk_idx = _c(topk_idx, np.int32)
    S, E = logits.shape
    k = topk_idx.shape[1]
    load = np.empty(E, np.float32); mp = np.empty(E, np.float32); aux = np.empty(1, np.float32)
    lib().orc_router_stats(_p(logits), _p(topk_idx), S, E, k, gate_fn, _p(load), _p(mp), _p(aux))
    return dict(load=load, mean_prob=mp, aux_loss=float(aux[0]))


def route_slots(topk_idx, E, drop, capacity):
    topk_idx = _c(topk_idx, np.int32)
    S, k = topk_idx.shape
    slot = np.empty((S, k), np.int32); cnt = np.empty(E, np.int32); off = np.empty(E, np.int32)
    tok = np.empty(S * k, np.int32); row = np.empty((S, k), np.int32)
    lib().orc_route(_p(topk_idx), S, k, E, drop, capacity, _p(slot), _p(cnt), _p(off), _p(tok), _p(row))
    return dict(slot=slot, expert_count=cnt, expert_offset=off, token_indices=tok, pair_row=row)


def route(cfg: Cfg, inp) -> dict:
    """Gate + top-k + slot assignment on all S tokens (cheap at every BASELINE size)."""
    logits = gate_logits(inp["x"], inp["gate_w"], inp.get("gate_bias"), cfg.act_dtype)
    idx, w = topk(logits, cfg.k, cfg.gate_fn, cfg.norm_topk)
    r = route_slots(idx, cfg.E, cfg.drop, cfg.capacity)
    r.update(logits=logits, topk_idx=idx, topk_w=w)
    return r


def gemm_bias_act(A, B, bias, dtype, act):
    M, K = A.shape; N = B.shape[0]
    out = np.empty((M, N), np.float32 if dtype in (F32, TF32) else np.uint16)
    lib().orc_gemm_bias_act(_p(np.ascontiguousarray(A)), _p(np.ascontiguousarray(B)),
                            _p(None if bias is None else np.ascontiguousarray(bias)), _p(out), M, N, K, dtype, act)
    return out


def expert_gemm(a_rows, w, bias, count, offset, dtype, act):
    """out[r] = act(a_rows[r] . w[e(r)]^T + bias[e(r)]) on packed expert-major rows; untouched rows are zero."""
    E, N, K = w.shape
    count = _c(count, np.int32); offset = _c(offset, np.int32)
    out = np.zeros((a_rows.shape[0], N), np.float32 if dtype in (F32, TF32) else np.uint16)
    lib().orc_expert_gemm(_p(np.ascontiguousarray(a_rows)), _p(np.ascontiguousarray(w)),
                          _p(None if bias is None else np.ascontiguousarray(bias)), _p(count), _p(offset), E, N, K,
                          dtype, act, _p(out))
    return out


def expert_wgrad(dy_rows, a_rows, count, offset, dtype):
    """dw[e] = sum over expert e's rows of dy_rows[r]^T a_rows[r] -> [E, N, K]."""
    count = _c(count, np.int32); offset = _c(offset, np.int32)
    N, K = dy_rows.shape[1], a_rows.shape[1]
    dw = np.empty((count.size, N, K), np.float32 if dtype in (F32, TF32) else np.uint16)
    lib().orc_expert_wgrad(_p(np.ascontiguousarray(dy_rows)), _p(np.ascontiguousarray(a_rows)), _p(count), _p(offset),
                           count.size, N, K, dtype, _p(dw))
    return dw


def act_backward(dh, u, g, dtype, act):
    """(du, dg): dg is None unless act is SwiGLU.  All arrays [rows, I] in the storage type."""
    rows, I = dh.shape
    du = np.empty_like(dh)
    dg = np.empty_like(dh) if act == ACT_SWIGLU else None
    lib().orc_act_backward(_p(np.ascontiguousarray(dh)), _p(np.ascontiguousarray(u)),
                           _p(None if g is None else np.ascontiguousarray(g)), rows, I, dtype, act, _p(du), _p(dg))
    return du, dg


def bias_grad(dy_rows, count, offset, dtype):
    count = _c(count, np.int32); offset = _c(offset, np.int32)
    db = np.empty((count.size, dy_rows.shape[1]), dy_rows.dtype)
    lib().orc_bias_grad(_p(np.ascontiguousarray(dy_rows)), _p(count), _p(offset), count.size, dy_rows.shape[1], dtype, _p(db))
    return db


def combine_backward(dout, y_rows, pair_row, topk_w, dtype):
    """(dy_rows [rows of y, H] with untouched rows zero, dw [S, k] fp32)."""
    pair_row = _c(pair_row, np.int32); topk_w = _c(topk_w, np.float32)
    S, k = pair_row.shape
    dy = np.zeros_like(y_rows)
    dw = np.empty((S, k), np.float32)
    lib().orc_combine_backward(_p(np.ascontiguousarray(dout)), _p(np.ascontiguousarray(y_rows)), _p(pair_row), _p(topk_w),
                               S, k, dout.shape[1], dtype, _p(dy), _p(dw))
    return dy, dw


def ffn_rows(cfg: Cfg, inp, tokens, experts):
    tokens = _c(tokens, np.int32); experts = _c(experts, np.int32)
    y = np.empty((tokens.size, cfg.H), np.float32 if cfg.act_dtype == F32 else np.uint16)
    cs, ws = cfg.c_struct(), _weights(inp)
    lib().orc_ffn_rows(C.byref(cs), _p(inp["x"]), C.byref(ws), _p(tokens), _p(experts), tokens.size, _p(y))
    return y


def combine(y_rows, pair_row, topk_w, H, act_dtype):
    pair_row = _c(pair_row, np.int32); topk_w = _c(topk_w, np.float32)
    S, k = pair_row.shape
    out = np.empty((S, H), np.float32 if act_dtype == F32 else np.uint16)
    lib().orc_combine(_p(np.ascontiguousarray(y_rows)), _p(pair_row), _p(topk_w), S, k, H, act_dtype, _p(out))
    return out


def forward(cfg: Cfg, inp) -> dict:
    S, k, E, H = cfg.S, cfg.k, cfg.E, cfg.H
    out = np.empty((S, H), np.float32 if cfg.act_dtype == F32 else np.uint16)
    idx = np.empty((S, k), np.int32); w = np.empty((S, k), np.float32); slot = np.empty((S, k), np.int32)
    cnt = np.empty(E, np.int32); off = np.empty(E, np.int32); tok = np.empty(S * k, np.int32)
    cs, ws = cfg.c_struct(), _weights(inp)
    lib().orc_forward(C.byref(cs), _p(inp["x"]), C.byref(ws), _p(out), _p(idx), _p(w), _p(slot), _p(cnt), _p(off),
                      _p(tok))
    return dict(out=out, topk_idx=idx, topk_w=w, slot=slot, expert_count=cnt, expert_offset=off, token_indices=tok)


def forward_tokens(cfg: Cfg, inp, topk_idx, topk_w, slot, tokens):
    tokens = _c(tokens, np.int32)
    topk_idx = _c(topk_idx, np.int32); topk_w = _c(topk_w, np.float32); slot = _c(slot, np.int32)
    out = np.empty((tokens.size, cfg.H), np.float32 if cfg.act_dtype == F32 else np.uint16)
    cs, ws = cfg.c_struct(), _weights(inp)
    lib().orc_forward_tokens(C.byref(cs), _p(inp["x"]), C.byref(ws), _p(topk_idx), _p(topk_w), _p(slot), _p(tokens),
                             tokens.size, _p(out))
    return out


def num_threads() -> int:
    return lib().orc_num_threads()
