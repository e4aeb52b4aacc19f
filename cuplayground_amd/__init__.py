"""moe355: MI355X (gfx950) fused MoE forward -- gate -> slot assignment -> expert FFN -> combine.

The product is `libmoe355.so` (C ABI in `include/moe355.h`, HIP kernels in `csrc/`).  This package is the
thin Python host side over that ABI: torch supplies device memory and the stream, nothing else.  There is no
fallback path: if the library is not built, importing `cuplayground_amd.api` symbols that need it raises.
`cuplayground_amd.torch_op` registers `torch.ops.moe355.forward`; `cuplayground_amd.weights` packs, quantises, saves and
loads a layer's weights in the operand layout.
"""
from .api import (  # noqa: F401
    MoEConfig,
    MoELayer,
    MoEError,
    combine,
    gemm_bias_act,
    library_path,
    load_library,
    measured_peaks,
    quantize_block128,
    quantize_rows128,
    dequantize_block128,
    transpose,
)
from . import api  # noqa: F401
