"""Builds libmoe355.so (host C++ + gfx950 HIP kernels) in-tree with hipcc."""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmoe355.so")
SOURCES = ["config.cpp", "api.hip", "gate.hip", "route.hip", "combine.hip", "ffn_bf16.hip", "ffn_f32.hip",
           "ffn_fp8.hip", "ffn_fp8_tile.hip", "ffn_f32_tile.hip", "peaks.hip", "quant.hip", "backward.hip"]
# packed-fp32 VALU forms are disabled for every device code object of this library
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-x", "hip", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         # the epilogues index the accumulator registers in fully unrolled loops; without this the 8 x 8 x 4 loop of
         # the large bf16 tile exceeds the default limit, stays rolled and sends the accumulators through memory
         "-mllvm", "-pragma-unroll-threshold=1000000"]


def _compile(src: str, extra) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = ["hipcc", *FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, r.stderr))
    noise = "'-packed-fp32-ops' is not a recognized feature"
    warn = "\n".join(l for l in r.stderr.splitlines() if l.strip() and noise not in l)
    if warn.strip():
        sys.stderr.write(warn + "\n")
    return obj


def build_library(extra_flags=(), jobs: int = 8) -> str:
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, list(extra_flags)), SOURCES))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build_library(sys.argv[1:]))
