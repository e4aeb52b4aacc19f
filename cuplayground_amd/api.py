"""ctypes binding of include/moe355.h plus a small host-side mirror of the operator.

`MoEConfig` carries exactly the keys of the reference's aristos_config.json (aristos_config.schema.json:5-58)
and this build's extensions; `MoELayer` owns a handle and a workspace tensor and calls `moe_forward`.
torch is used for device memory and the current HIP stream only.
"""
from __future__ import annotations

import ctypes as C
import json
import os
from dataclasses import asdict, dataclass

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmoe355.so")

DTYPE_F32, DTYPE_TF32, DTYPE_BF16, DTYPE_FP16, DTYPE_FP8 = 0, 1, 2, 3, 4
ACT_RELU, ACT_GELU, ACT_SWIGLU, ACT_NONE = 0, 1, 2, 3
GATE_SOFTMAX, GATE_SIGMOID = 0, 1
FFN_AUTO, FFN_TILED, FFN_PERSISTENT = 0, 1, 2
STAGES = ("gate", "route", "ffn", "combine")

EXPORTS = (
    "moe_config_default", "moe_config_from_json_string", "moe_config_from_json_file", "moe_config_validate",
    "moe_config_tokens", "moe_config_capacity", "moe_create", "moe_destroy", "moe_get_arch", "moe_get_plan", "moe_get_kernel_dtype",
    "moe_workspace_bytes", "moe_options_default", "moe_options_from_env", "moe_create_with_options",
    "moe_workspace_bytes_with_options", "moe_get_options", "moe_get_workspace_bytes", "moe_get_stall", "moe_gemm_bias_act_tile",
    "moe_prepared_bytes", "moe_prepare_weights", "moe_quant_rows128",
    "moe_set_ffn_mode", "moe_get_ffn_mode", "moe_forward", "moe_forward_static", "moe_set_spin_limit", "moe_clear_stall", "moe_gate", "moe_router_stats", "moe_route", "moe_gemm_bias_act", "moe_combine",
    "moe_set_stage_timing", "moe_get_stage_ms", "moe_get_stage_samples", "moe_get_task_counts", "moe_get_queue_balance", "moe_task_trace_bytes", "moe_set_task_trace", "moe_get_task_trace", "moe_measure_mfma_tflops",
    "moe_measure_hbm_read_gbs", "moe_quant_block128", "moe_dequant_block128", "moe_backward_scratch_bytes", "moe_transpose", "moe_expert_gemm",
    "moe_expert_gemm_act_backward", "moe_expert_gemm_act_backward_supported", "moe_expert_wgrad", "moe_act_backward", "moe_bias_grad", "moe_combine_backward", "moe_last_hip_error", "moe_status_string",
    "moe_version",
)


class MoEError(RuntimeError):
    def __init__(self, status: int, what: str = ""):
        self.status = status
        msg = load_library().moe_status_string(status).decode()
        super().__init__("moe355 status %d (%s)%s" % (status, msg, (": " + what) if what else ""))


class _CConfig(C.Structure):
    _fields_ = [("capacity_factor", C.c_double)] + [(n, C.c_int32) for n in (
        "drop_tokens", "expert_top_k", "is_training", "hidden_act", "hidden_size", "intermediate_size", "micro_batch",
        "num_experts", "sequence_len", "torch_dtype", "gate_fn", "norm_topk_prob")]


OPTION_FIELDS = ("tile16", "block_rows", "f32_tile", "fp8_tile", "fp8_widen", "queue_groups", "queue_lag", "queue_early",
                 "row_chunk", "blocks_per_cu", "combine", "gate_kernel", "gate_mfma", "gate_tile", "gate_fused_topk",
                 "grouped_tile", "tail_round", "fp8_mfma", "prepared_weights", "tail_split")
OPT_AUTO = -1
COMBINE_SEPARATE, COMBINE_ARRIVALS, COMBINE_QUEUE = 0, 1, 2


class _COptions(C.Structure):
    _fields_ = [(n, C.c_int32) for n in OPTION_FIELDS] + [("reserved", C.c_int32 * 6)]


def make_options(options: dict | None = None, from_env: bool = False) -> _COptions:
    """moe_options with every field AUTO, then (from_env) the MOE355_* variables, then `options` (field name -> int)."""
    L = load_library()
    o = _COptions()
    _check(L.moe_options_default(C.byref(o)))
    if from_env:
        _check(L.moe_options_from_env(C.byref(o)))
    for k, v in (options or {}).items():
        if k not in OPTION_FIELDS:
            raise KeyError("unknown option %r (known: %s)" % (k, ", ".join(OPTION_FIELDS)))
        setattr(o, k, int(v))
    return o


class _CArch(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("device", "compute_units", "xcds", "wavefront_size", "lds_bytes_per_cu",
                                         "max_clock_khz", "persistent_blocks")] + [("name", C.c_char * 64)]


class _CWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("gate_w", "gate_bias", "w_up", "w_gate", "w_down", "b_up", "b_gate",
                                          "b_down", "s_up", "s_gate", "s_down", "prepared")]


class _CRouting(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("topk_idx", "topk_w", "slot", "expert_count", "expert_offset",
                                          "token_indices")]


_lib = None


def library_path() -> str:
    return _LIB_PATH


def load_library():
    """Loads libmoe355.so; raises if it has not been built (there is no other implementation to fall back to)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError("libmoe355.so is not built: run `python -m cuplayground_amd.build` (needs hipcc)")
    L = C.CDLL(_LIB_PATH)
    vp, i32, i64 = C.c_void_p, C.c_int32, C.c_int64
    cfgp = C.POINTER(_CConfig)
    L.moe_config_default.argtypes = [cfgp]
    L.moe_config_from_json_string.argtypes = [C.c_char_p, cfgp, C.c_char_p, C.c_size_t]
    L.moe_config_from_json_file.argtypes = [C.c_char_p, cfgp, C.c_char_p, C.c_size_t]
    L.moe_config_validate.argtypes = [cfgp, C.c_char_p, C.c_size_t]
    L.moe_config_tokens.argtypes = [cfgp]; L.moe_config_tokens.restype = i64
    L.moe_config_capacity.argtypes = [cfgp, C.POINTER(i64)]
    L.moe_create.argtypes = [cfgp, C.POINTER(vp)]
    L.moe_destroy.argtypes = [vp]
    L.moe_get_arch.argtypes = [vp, C.POINTER(_CArch)]
    L.moe_get_plan.argtypes = [vp, C.POINTER(i32), C.POINTER(i32), C.POINTER(i32)]
    L.moe_get_kernel_dtype.argtypes = [vp, C.POINTER(i32)]
    L.moe_workspace_bytes.argtypes = [cfgp, C.POINTER(C.c_size_t)]
    optp = C.POINTER(_COptions)
    L.moe_options_default.argtypes = [optp]
    L.moe_options_from_env.argtypes = [optp]
    L.moe_create_with_options.argtypes = [cfgp, optp, C.POINTER(vp)]
    L.moe_workspace_bytes_with_options.argtypes = [cfgp, optp, C.POINTER(C.c_size_t)]
    L.moe_get_options.argtypes = [vp, optp]
    L.moe_get_workspace_bytes.argtypes = [vp, C.POINTER(C.c_size_t)]
    L.moe_get_stall.argtypes = [vp, C.POINTER(i32)]
    L.moe_prepared_bytes.argtypes = [vp, C.POINTER(C.c_size_t)]
    L.moe_prepare_weights.argtypes = [vp, C.POINTER(_CWeights), vp, C.c_size_t, vp]
    L.moe_gemm_bias_act_tile.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32, i32, vp]
    L.moe_set_ffn_mode.argtypes = [vp, C.c_int]
    L.moe_get_ffn_mode.argtypes = [vp, C.POINTER(C.c_int32)]
    L.moe_forward.argtypes = [vp, vp, C.POINTER(_CWeights), vp, C.POINTER(_CRouting), vp, C.c_size_t, vp]
    L.moe_forward_static.argtypes = [vp, vp, C.POINTER(_CWeights), vp, C.POINTER(_CRouting), vp]
    L.moe_set_spin_limit.argtypes = [vp, i32]
    L.moe_clear_stall.argtypes = [vp]
    L.moe_router_stats.argtypes = [vp, vp, vp, vp, vp, vp, vp, C.c_size_t, vp]
    L.moe_gate.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, C.c_size_t, vp]
    L.moe_route.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, C.c_size_t, vp]
    L.moe_gemm_bias_act.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32, vp]
    L.moe_combine.argtypes = [vp, vp, vp, i32, i32, i32, i32, vp, vp]
    L.moe_set_stage_timing.argtypes = [vp, C.c_int]
    L.moe_get_stage_ms.argtypes = [vp, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_int32)]
    L.moe_get_stage_samples.argtypes = [vp, C.c_int, C.POINTER(C.c_float), C.c_int32, C.POINTER(C.c_int32)]
    L.moe_get_task_counts.argtypes = [vp, vp, vp, C.POINTER(i64), C.POINTER(i64)]
    L.moe_get_queue_balance.argtypes = [vp, vp, vp, C.POINTER(i32), C.POINTER(C.c_float), C.POINTER(C.c_float),
                                        C.POINTER(C.c_float)]
    L.moe_task_trace_bytes.argtypes = [C.c_int64]
    L.moe_task_trace_bytes.restype = C.c_size_t
    L.moe_set_task_trace.argtypes = [vp, vp, C.c_size_t]
    L.moe_get_task_trace.argtypes = [vp, vp, vp, C.c_int64, C.POINTER(C.c_int64)]
    L.moe_quant_block128.argtypes = [vp, C.c_int32, C.c_int64, C.c_int64, C.c_int64, vp, vp, vp]
    L.moe_dequant_block128.argtypes = [vp, vp, C.c_int64, C.c_int64, C.c_int64, vp, vp]
    L.moe_quant_rows128.argtypes = [vp, C.c_int64, C.c_int64, vp, vp, vp]
    L.moe_measure_mfma_tflops.argtypes = [vp, C.c_size_t, vp, C.c_int, C.POINTER(C.c_float)]
    L.moe_measure_hbm_read_gbs.argtypes = [vp, C.c_size_t, vp, vp, C.POINTER(C.c_float)]
    L.moe_backward_scratch_bytes.argtypes = [cfgp, C.POINTER(C.c_size_t)]
    L.moe_transpose.argtypes = [vp, vp, i64, i64, i64, i32, vp]
    L.moe_expert_gemm.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, vp, vp, C.c_size_t, vp]
    L.moe_expert_wgrad.argtypes = [vp, vp, vp, vp, vp, i32, i32, vp, vp, C.c_size_t, vp]
    L.moe_expert_gemm_act_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32, vp, vp, vp, C.c_size_t, vp]
    L.moe_expert_gemm_act_backward_supported.argtypes = [vp, C.POINTER(C.c_int32)]
    L.moe_act_backward.argtypes = [vp, vp, vp, vp, i64, vp, vp, vp]
    L.moe_bias_grad.argtypes = [vp, vp, vp, vp, i32, vp, vp]
    L.moe_combine_backward.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp]
    L.moe_last_hip_error.argtypes = [vp]
    L.moe_status_string.argtypes = [C.c_int]; L.moe_status_string.restype = C.c_char_p
    L.moe_version.restype = C.c_int
    _lib = L
    return L


def _check(rc: int, what: str = ""):
    if rc != 0:
        raise MoEError(rc, what)


@dataclass
class MoEConfig:
    """The operator's knobs; names and meanings are those of aristos_config.json."""
    capacity_factor: float = 1.0
    drop_tokens: int = 0
    expert_top_k: int = 1
    is_training: int = 0
    hidden_act: int = ACT_RELU
    hidden_size: int = 1024
    intermediate_size: int = 4096
    micro_batch: int = 4
    num_experts: int = 1
    sequence_len: int = 2048
    torch_dtype: int = DTYPE_F32
    gate_fn: int = GATE_SOFTMAX
    norm_topk_prob: int = 0

    def to_c(self) -> _CConfig:
        return _CConfig(float(self.capacity_factor), *[int(getattr(self, n)) for n, _ in _CConfig._fields_[1:]])

    @classmethod
    def _from_c(cls, c: _CConfig) -> "MoEConfig":
        return cls(**{n: getattr(c, n) for n, _ in _CConfig._fields_})

    @classmethod
    def from_json(cls, text_or_path: str) -> "MoEConfig":
        """Parses and validates with the library's own loader (the same one a C caller gets)."""
        L = load_library()
        c = _CConfig()
        err = C.create_string_buffer(256)
        if os.path.exists(text_or_path):
            rc = L.moe_config_from_json_file(text_or_path.encode(), C.byref(c), err, len(err))
        else:
            rc = L.moe_config_from_json_string(text_or_path.encode(), C.byref(c), err, len(err))
        _check(rc, err.value.decode())
        return cls._from_c(c)

    def to_json(self) -> str:
        return json.dumps(asdict(self), indent=2)

    def validate(self) -> None:
        err = C.create_string_buffer(256)
        c = self.to_c()
        _check(load_library().moe_config_validate(C.byref(c), err, len(err)), err.value.decode())

    @property
    def tokens(self) -> int:
        return self.micro_batch * self.sequence_len

    @property
    def capacity(self) -> int:
        out = C.c_int64(0)
        c = self.to_c()
        _check(load_library().moe_config_capacity(C.byref(c), C.byref(out)))
        return out.value

    def workspace_bytes(self) -> int:
        out = C.c_size_t(0)
        c = self.to_c()
        _check(load_library().moe_workspace_bytes(C.byref(c), C.byref(out)))
        return out.value


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _torch_act_dtype(torch_dtype: int):
    """Storage type of activations: the layer's own; fp32 for tf32 layers, bf16 for e4m3 layers."""
    import torch
    if torch_dtype in (DTYPE_F32, DTYPE_TF32):
        return torch.float32
    return torch.float16 if torch_dtype == DTYPE_FP16 else torch.bfloat16


class MoELayer:
    """One MoE layer shape bound to the current GPU: a `moe_handle` and its workspace."""

    WEIGHT_KEYS = ("gate_w", "gate_bias", "w_up", "w_gate", "w_down", "b_up", "b_gate", "b_down", "s_up", "s_gate",
                   "s_down", "prepared")

    def __init__(self, cfg: MoEConfig, ffn_mode: int = FFN_AUTO, allocate_workspace: bool = True,
                 options: dict | None = None):
        """options: tuning options by field name of moe_options (e.g. {"tile16": 1, "combine": 2}); None creates the
        handle with moe_create, i.e. library defaults overridden by MOE355_* environment variables."""
        import torch
        self.cfg = cfg
        self.L = load_library()
        self._h = C.c_void_p()
        c = cfg.to_c()
        if options is None:
            _check(self.L.moe_create(C.byref(c), C.byref(self._h)), "moe_create")
        else:
            o = make_options(options)
            _check(self.L.moe_create_with_options(C.byref(c), C.byref(o), C.byref(self._h)), "moe_create_with_options")
        n = C.c_size_t(0)
        _check(self.L.moe_get_workspace_bytes(self._h, C.byref(n)), "moe_get_workspace_bytes")
        self.workspace_bytes = n.value
        # allocate_workspace=False: for callers that only use forward(static_workspace=True)
        self.workspace = (torch.empty(self.workspace_bytes, dtype=torch.uint8, device="cuda")
                          if allocate_workspace else None)
        self.S, self.k, self.E, self.H = cfg.tokens, cfg.expert_top_k, cfg.num_experts, cfg.hidden_size
        self.act_dtype = _torch_act_dtype(cfg.torch_dtype)
        if ffn_mode != FFN_AUTO:
            self.set_ffn_mode(ffn_mode)

    def close(self):
        if getattr(self, "_h", None) is not None and self._h:
            self.L.moe_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def arch(self) -> dict:
        a = _CArch()
        _check(self.L.moe_get_arch(self._h, C.byref(a)))
        d = {n: getattr(a, n) for n, _ in _CArch._fields_}
        d["name"] = a.name.decode()
        return d

    @property
    def plan(self) -> dict:
        a, b, c = C.c_int32(0), C.c_int32(0), C.c_int32(0)
        _check(self.L.moe_get_plan(self._h, C.byref(a), C.byref(b), C.byref(c)))
        return dict(block_rows=a.value, col_tiles_up=b.value, col_tiles_down=c.value)

    @property
    def kernel_dtype(self) -> int:
        """The dtype whose FFN kernels run: the layer's own, or DTYPE_BF16 for an e4m3 layer with so many rows per
        expert that every call widens the weights into the workspace and runs the bf16 tiles."""
        d = C.c_int32(0)
        _check(self.L.moe_get_kernel_dtype(self._h, C.byref(d)))
        return d.value

    @property
    def options(self) -> dict:
        """The options in force, every AUTO the library could resolve at creation replaced by its choice."""
        o = _COptions()
        _check(self.L.moe_get_options(self._h, C.byref(o)))
        return {n: getattr(o, n) for n in OPTION_FIELDS}

    @property
    def stalled(self) -> bool:
        v = C.c_int32(0)
        _check(self.L.moe_get_stall(self._h, C.byref(v)))
        return bool(v.value)

    def set_ffn_mode(self, mode: int):
        _check(self.L.moe_set_ffn_mode(self._h, mode))

    @property
    def ffn_mode(self) -> int:
        """The FFN variant forward() runs: 1 = one launch per projection, 2 = task queue."""
        m = C.c_int32(0)
        _check(self.L.moe_get_ffn_mode(self._h, C.byref(m)))
        return m.value

    def set_stage_timing(self, enable: bool):
        _check(self.L.moe_set_stage_timing(self._h, int(enable)))

    def stage_ms(self) -> dict:
        """Mean milliseconds per stage over the forward calls recorded since set_stage_timing(True)."""
        out = {}
        calls = C.c_int32(0)
        for i, n in enumerate(STAGES):
            v = C.c_float(0)
            _check(self.L.moe_get_stage_ms(self._h, i, C.byref(v), C.byref(calls)))
            out[n] = v.value
        out["calls"] = calls.value
        return out

    def stage_samples(self) -> dict:
        """Per-call milliseconds of every stage and of the whole call ("total") for the most recent recorded calls
        (64 at most), oldest first."""
        out = {}
        buf = (C.c_float * 64)()
        n = C.c_int32(0)
        for i, name in enumerate(STAGES + ("total",)):
            _check(self.L.moe_get_stage_samples(self._h, i, buf, 64, C.byref(n)))
            out[name] = [buf[j] for j in range(n.value)]
        return out

    def task_counts(self):
        """(up-projection tasks, down-projection tasks) of the last forward; without a workspace of its own the layer
        reads the library's static array (the last forward(static_workspace=True))."""
        a, b = C.c_int64(0), C.c_int64(0)
        _check(self.L.moe_get_task_counts(self._h, _ptr(self.workspace), _stream(), C.byref(a), C.byref(b)))
        return a.value, b.value

    def queue_balance(self) -> dict:
        """Workgroup entry/exit statistics of the last forward's queue kernel (microseconds)."""
        n, a, b, c = C.c_int32(0), C.c_float(0), C.c_float(0), C.c_float(0)
        _check(self.L.moe_get_queue_balance(self._h, _ptr(self.workspace), _stream(), C.byref(n), C.byref(a),
                                            C.byref(b), C.byref(c)), "moe_get_queue_balance")
        return dict(workgroups=n.value, span_us=a.value, mean_active_us=b.value, mean_tail_idle_us=c.value)

    def enable_task_trace(self, max_tasks: int = 1 << 16):
        """Every task of the queue kernel leaves a record from now on (see task_trace); the buffer is a torch tensor."""
        import torch
        nbytes = self.L.moe_task_trace_bytes(max_tasks)
        self._trace = torch.zeros(nbytes // 8, dtype=torch.int64, device="cuda")
        torch.cuda.synchronize()
        _check(self.L.moe_set_task_trace(self._h, _ptr(self._trace), nbytes), "moe_set_task_trace")

    def disable_task_trace(self):
        _check(self.L.moe_set_task_trace(self._h, None, 0), "moe_set_task_trace")
        self._trace = None

    def task_trace(self):
        """Records of the last forward's queue kernel as a numpy structured array (phase, expert, row_block, col_tile,
        rows, workgroup, start_us, end_us); synchronises the current stream.  A task that computed one of P partial sums of
        its tile (option tail_split) carries 1 + 4 * part + 16 * P in `phase`."""
        import numpy as np
        dt = np.dtype([("phase", "i4"), ("expert", "i4"), ("row_block", "i4"), ("col_tile", "i4"), ("rows", "i4"),
                       ("workgroup", "i4"), ("start_us", "f4"), ("end_us", "f4")])
        n = C.c_int64(0)
        _check(self.L.moe_get_task_trace(self._h, _stream(), None, 0, C.byref(n)), "moe_get_task_trace")
        out = np.zeros(n.value, dtype=dt)
        if n.value:
            _check(self.L.moe_get_task_trace(self._h, _stream(), out.ctypes.data, n.value, C.byref(n)), "moe_get_task_trace")
        return out

    def _weights(self, weights: dict) -> _CWeights:
        w = _CWeights()
        for n in self.WEIGHT_KEYS:
            t = weights.get(n)
            setattr(w, n, None if t is None else t.data_ptr())
        return w

    @property
    def prepared_bytes(self) -> int:
        """Bytes moe_prepare_weights writes for this handle's plan (0: the plan reads the weights as they are)."""
        n = C.c_size_t(0)
        _check(self.L.moe_prepared_bytes(self._h, C.byref(n)), "moe_prepared_bytes")
        return n.value

    def prepare_weights(self, weights: dict, out=None):
        """The kernel-ready form of `weights` for this handle (a uint8 tensor to pass on as weights["prepared"]), or
        None when the plan prepares nothing.  `out`: a tensor of prepared_bytes bytes to write into (e.g. one loaded
        from a file's worth of storage); allocated when not given."""
        import torch
        n = self.prepared_bytes
        if n == 0:
            return None
        if out is None:
            out = torch.empty(n, dtype=torch.uint8, device="cuda")
        w = self._weights(weights)
        _check(self.L.moe_prepare_weights(self._h, C.byref(w), _ptr(out), out.numel() * out.element_size(), _stream()),
               "moe_prepare_weights")
        return out

    def new_routing(self) -> dict:
        import torch
        dev = "cuda"
        S, k, E = self.S, self.k, self.E
        return dict(topk_idx=torch.empty(S, k, dtype=torch.int32, device=dev),
                    topk_w=torch.empty(S, k, dtype=torch.float32, device=dev),
                    slot=torch.empty(S, k, dtype=torch.int32, device=dev),
                    expert_count=torch.empty(E, dtype=torch.int32, device=dev),
                    expert_offset=torch.empty(E, dtype=torch.int32, device=dev),
                    token_indices=torch.empty(S * k, dtype=torch.int32, device=dev))

    def forward(self, x, weights: dict, out=None, routing: dict | None = None, static_workspace: bool = False):
        """out[S,H] = MoE(x).  `routing` (from new_routing()) receives the routing result when given.
        static_workspace: call moe_forward_static (the library's own per-GPU array instead of self.workspace)."""
        import torch
        if out is None:
            out = torch.empty(self.S, self.H, dtype=self.act_dtype, device=x.device)
        w = self._weights(weights)
        r = None
        if routing is not None:
            r = _CRouting(*[routing[n].data_ptr() for n, _ in _CRouting._fields_])
        rp = C.byref(r) if r is not None else None
        if static_workspace:
            _check(self.L.moe_forward_static(self._h, _ptr(x), C.byref(w), _ptr(out), rp, _stream()),
                   "moe_forward_static")
        else:
            _check(self.L.moe_forward(self._h, _ptr(x), C.byref(w), _ptr(out), rp, _ptr(self.workspace),
                                      self.workspace_bytes, _stream()), "moe_forward")
        return out

    def set_spin_limit(self, polls: int):
        """Polls before a dependency wait of the queue kernel gives up (0: default; negative: every wait expires)."""
        _check(self.L.moe_set_spin_limit(self._h, polls))

    def clear_stall(self):
        _check(self.L.moe_clear_stall(self._h))

    def gate(self, x, gate_w, gate_bias=None, want_logits: bool = False):
        import torch
        idx = torch.empty(self.S, self.k, dtype=torch.int32, device=x.device)
        wts = torch.empty(self.S, self.k, dtype=torch.float32, device=x.device)
        logits = torch.empty(self.S, self.E, dtype=torch.float32, device=x.device) if want_logits else None
        _check(self.L.moe_gate(self._h, _ptr(x), _ptr(gate_w), _ptr(gate_bias), _ptr(logits), _ptr(idx), _ptr(wts),
                               _ptr(self.workspace), self.workspace_bytes, _stream()), "moe_gate")
        return (idx, wts, logits) if want_logits else (idx, wts)

    def router_stats(self, logits, topk_idx) -> dict:
        """load[E], mean_prob[E] and aux_loss (a 1-element tensor) from the router's logits and choices."""
        import torch
        dev = logits.device
        out = dict(load=torch.empty(self.E, dtype=torch.float32, device=dev),
                   mean_prob=torch.empty(self.E, dtype=torch.float32, device=dev),
                   aux_loss=torch.empty(1, dtype=torch.float32, device=dev))
        _check(self.L.moe_router_stats(self._h, _ptr(logits), _ptr(topk_idx), _ptr(out["load"]), _ptr(out["mean_prob"]),
                                       _ptr(out["aux_loss"]), _ptr(self.workspace), self.workspace_bytes, _stream()),
               "moe_router_stats")
        return out

    def route(self, topk_idx):
        import torch
        dev = topk_idx.device
        S, k, E = self.S, self.k, self.E
        r = dict(slot=torch.empty(S, k, dtype=torch.int32, device=dev),
                 expert_count=torch.empty(E, dtype=torch.int32, device=dev),
                 expert_offset=torch.empty(E, dtype=torch.int32, device=dev),
                 token_indices=torch.empty(S * k, dtype=torch.int32, device=dev),
                 pair_row=torch.empty(S, k, dtype=torch.int32, device=dev))
        _check(self.L.moe_route(self._h, _ptr(topk_idx), _ptr(r["slot"]), _ptr(r["expert_count"]),
                                _ptr(r["expert_offset"]), _ptr(r["token_indices"]), _ptr(r["pair_row"]),
                                _ptr(self.workspace), self.workspace_bytes, _stream()), "moe_route")
        return r

    # ---- backward building blocks (fp32, bf16 and fp16 layers) ----
    def backward_scratch(self):
        """Device scratch for expert_gemm / expert_wgrad, allocated on first use and kept with the layer."""
        import torch
        if getattr(self, "_bwd_scratch", None) is None:
            n = C.c_size_t(0)
            _check(self.L.moe_backward_scratch_bytes(C.byref(self.cfg.to_c()), C.byref(n)), "moe_backward_scratch_bytes")
            self._bwd_scratch = torch.empty(n.value, dtype=torch.uint8, device="cuda")
        return self._bwd_scratch

    def expert_gemm(self, a_rows, w, bias, expert_count, expert_offset, act: int = ACT_NONE, out=None):
        """out_rows[r] = act(a_rows[r] . w[e(r)]^T + bias[e(r)]) over the kept packed rows; w [E,N,K]."""
        import torch
        N, K = w.shape[1], w.shape[2]
        if out is None:
            out = torch.zeros(a_rows.shape[0], N, dtype=a_rows.dtype, device=a_rows.device)
        sc = self.backward_scratch()
        _check(self.L.moe_expert_gemm(self._h, _ptr(a_rows), _ptr(w), _ptr(bias), _ptr(expert_count),
                                      _ptr(expert_offset), N, K, act, _ptr(out), _ptr(sc), sc.numel(), _stream()),
               "moe_expert_gemm")
        return out

    @property
    def fused_act_backward(self) -> bool:
        """Whether expert_gemm_act_backward exists for this layer (16-bit, shape fit for the hand-ordered tiles)."""
        v = C.c_int32(0)
        _check(self.L.moe_expert_gemm_act_backward_supported(self._h, C.byref(v)))
        return bool(v.value)

    def expert_gemm_act_backward(self, dy_rows, w_down_t, u_rows, g_rows, expert_count, expert_offset, du=None, dg=None):
        """(du_rows, dg_rows) = (dy_rows . w_down_t[e(r)]^T) * act'(u_rows, g_rows): the data gradient of the down
        projection and the activation's derivative in one kernel; w_down_t [E, I, H]; dg_rows is None unless SwiGLU.
        Rows of no expert are not written (zeros in the buffers made here)."""
        import torch
        N, K = w_down_t.shape[1], w_down_t.shape[2]
        if du is None:
            du = torch.zeros(dy_rows.shape[0], N, dtype=dy_rows.dtype, device=dy_rows.device)
        if dg is None and g_rows is not None:
            dg = torch.zeros_like(du)
        sc = self.backward_scratch()
        _check(self.L.moe_expert_gemm_act_backward(self._h, _ptr(dy_rows), _ptr(w_down_t), _ptr(u_rows), _ptr(g_rows),
                                                   _ptr(expert_count), _ptr(expert_offset), N, K, _ptr(du), _ptr(dg),
                                                   _ptr(sc), sc.numel(), _stream()), "moe_expert_gemm_act_backward")
        return du, dg

    def expert_wgrad(self, dy_rows, a_rows, expert_count, expert_offset, out=None):
        """dw[e] [N,K] = sum over expert e's rows of dy_rows[r,:N]^T a_rows[r,:K]."""
        import torch
        N, K = dy_rows.shape[1], a_rows.shape[1]
        if out is None:
            out = torch.empty(self.E, N, K, dtype=a_rows.dtype, device=a_rows.device)
        sc = self.backward_scratch()
        _check(self.L.moe_expert_wgrad(self._h, _ptr(dy_rows), _ptr(a_rows), _ptr(expert_count), _ptr(expert_offset),
                                       N, K, _ptr(out), _ptr(sc), sc.numel(), _stream()), "moe_expert_wgrad")
        return out

    def act_backward(self, dh_rows, u_rows, g_rows=None, du=None, dg=None):
        """(du_rows, dg_rows) for the layer's activation; dg_rows is None unless the layer is SwiGLU."""
        import torch
        if du is None:
            du = torch.empty_like(dh_rows)
        if dg is None and g_rows is not None:
            dg = torch.empty_like(dh_rows)
        _check(self.L.moe_act_backward(self._h, _ptr(dh_rows), _ptr(u_rows), _ptr(g_rows), dh_rows.shape[0], _ptr(du),
                                       _ptr(dg), _stream()), "moe_act_backward")
        return du, dg

    def bias_grad(self, dy_rows, expert_count, expert_offset):
        import torch
        db = torch.empty(self.E, dy_rows.shape[1], dtype=dy_rows.dtype, device=dy_rows.device)
        _check(self.L.moe_bias_grad(self._h, _ptr(dy_rows), _ptr(expert_count), _ptr(expert_offset), dy_rows.shape[1],
                                    _ptr(db), _stream()), "moe_bias_grad")
        return db

    def combine_backward(self, dout, y_rows, pair_row, topk_w):
        """(dy_rows with the rows no pair maps to zero, dw [S, k] fp32)."""
        import torch
        dy = torch.zeros_like(y_rows)
        dw = torch.empty(self.S, self.k, dtype=torch.float32, device=dout.device)
        _check(self.L.moe_combine_backward(self._h, _ptr(dout), _ptr(y_rows), _ptr(pair_row), _ptr(topk_w), _ptr(dy),
                                           _ptr(dw), _stream()), "moe_combine_backward")
        return dy, dw


def transpose(src, out=None):
    """[.., R, C] -> [.., C, R] for 2- and 4-byte element types, batched over the leading dimensions."""
    import torch
    R, Cc = src.shape[-2], src.shape[-1]
    src = src.contiguous()
    if out is None:
        out = torch.empty(*src.shape[:-2], Cc, R, dtype=src.dtype, device=src.device)
    _check(load_library().moe_transpose(_ptr(src), _ptr(out), src.numel() // (R * Cc), R, Cc, src.element_size(),
                                        _stream()), "moe_transpose")
    return out


def measured_peaks() -> dict:
    """bf16 MFMA issue rate (TFLOP/s; zero and random operands) and streaming read bandwidth (GB/s) of this device."""
    import torch
    L = load_library()
    buf = torch.zeros(2 << 30, dtype=torch.uint8, device="cuda")
    scratch = torch.zeros(4 << 20, dtype=torch.uint8, device="cuda")
    tf, tfr, gb = C.c_float(0), C.c_float(0), C.c_float(0)
    _check(L.moe_measure_mfma_tflops(_ptr(scratch), scratch.numel(), _stream(), 0, C.byref(tf)), "moe_measure_mfma_tflops")
    _check(L.moe_measure_mfma_tflops(_ptr(scratch), scratch.numel(), _stream(), 1, C.byref(tfr)), "moe_measure_mfma_tflops")
    _check(L.moe_measure_hbm_read_gbs(_ptr(buf), buf.numel(), _ptr(scratch), _stream(), C.byref(gb)),
           "moe_measure_hbm_read_gbs")
    del buf
    return {"mfma_bf16_tflops": tf.value, "mfma_bf16_tflops_random_operands": tfr.value, "hbm_read_gbs": gb.value}


def quantize_block128(w):
    """[.., N, K] fp32/bf16 weights on the GPU -> (uint8 e4m3 codes of the same shape, fp32 scales [.., N/128, K/128])."""
    import torch
    N, K = w.shape[-2], w.shape[-1]
    mats = w.numel() // (N * K)
    w = w.contiguous()
    q = torch.empty(w.shape, dtype=torch.uint8, device=w.device)
    s = torch.empty(*w.shape[:-2], N // 128, K // 128, dtype=torch.float32, device=w.device)
    dtype = DTYPE_F32 if w.dtype == torch.float32 else DTYPE_BF16
    if w.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("quantize_block128 takes fp32 or bf16 weights")
    _check(load_library().moe_quant_block128(_ptr(w), dtype, mats, N, K, _ptr(q), _ptr(s), _stream()),
           "moe_quant_block128")
    return q, s


def quantize_rows128(x):
    """bf16 rows [R, K] on the GPU -> (uint8 e4m3 codes [R, K], fp32 scales [R, K/128]): one scale per row and 128 columns,
    the activation format of the e4m3 x e4m3 plan (option fp8_mfma)."""
    import torch
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        raise ValueError("quantize_rows128 takes a 2-d bf16 tensor")
    x = x.contiguous()
    R, K = x.shape
    q = torch.empty(R, K, dtype=torch.uint8, device=x.device)
    s = torch.empty(R, K // 128, dtype=torch.float32, device=x.device)
    _check(load_library().moe_quant_rows128(_ptr(x), R, K, _ptr(q), _ptr(s), _stream()), "moe_quant_rows128")
    return q, s


def dequantize_block128(q, s):
    """bf16(e4m3(q) * scale of its 128x128 block), rounded once: what an e4m3 layer with many rows per expert runs its
    bf16 tile GEMM on.  q: uint8 / float8_e4m3fn [..., N, K], s: fp32 [..., N/128, K/128]."""
    import torch
    N, K = q.shape[-2:]
    mats = q.numel() // (N * K)
    q = q.contiguous()
    s = s.contiguous()
    out = torch.empty(q.shape, dtype=torch.bfloat16, device=q.device)
    _check(load_library().moe_dequant_block128(_ptr(q), _ptr(s), mats, N, K, _ptr(out), _stream()),
           "moe_dequant_block128")
    return out


def gemm_bias_act(A, B, bias, act: int, tile: int = OPT_AUTO):
    """C = act(A.B^T + bias): the reference tile GEMM contract (mma.cuh:46-179) on dense operands.
    tile: OPT_AUTO, or the tile of moe_gemm_bias_act_tile."""
    import torch
    M, K = A.shape
    N = B.shape[0]
    dtype = {torch.float32: DTYPE_F32, torch.bfloat16: DTYPE_BF16, torch.float16: DTYPE_FP16}[A.dtype]
    Cm = torch.empty(M, N, dtype=A.dtype, device=A.device)
    _check(load_library().moe_gemm_bias_act_tile(_ptr(A), _ptr(B), _ptr(bias), _ptr(Cm), M, N, K, dtype, act, tile,
                                                 _stream()), "moe_gemm_bias_act_tile")
    return Cm


def combine(y_rows, pair_row, topk_w, out=None):
    """out[t,:] = sum_r w[t,r] * y_rows[pair_row[t,r],:] (combine.cuh:170-186 in gather form)."""
    import torch
    S, k = pair_row.shape
    H = y_rows.shape[1]
    dtype = {torch.float32: DTYPE_F32, torch.bfloat16: DTYPE_BF16, torch.float16: DTYPE_FP16}[y_rows.dtype]
    if out is None:
        out = torch.empty(S, H, dtype=y_rows.dtype, device=y_rows.device)
    _check(load_library().moe_combine(_ptr(y_rows), _ptr(pair_row), _ptr(topk_w), S, k, H, dtype, _ptr(out),
                                      _stream()), "moe_combine")
    return out
