"""Compile the HIP sources under csrc/ into turboquant_amd/libtq_hip.so for gfx950.

hipcc cross-compiles without a GPU, so this runs in the build container; the
shared object is loaded by `_ffi.py` and is never built implicitly at import.
"""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libtq_hip.so")
SOURCES = ["tq_quantize.hip", "tq_quantize_mfma.hip", "tq_score.hip", "tq_decode.hip", "tq_decode_mfma.hip", "tq_probe.hip"]

# packed-fp32 instructions stay off: some of their forms have produced wrong
# results on this hardware pool
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no implicit a*b+c fusion: the quantisers mirror separately rounded torch ops;
    # the kernels call fmaf() explicitly wherever a fused multiply-add is wanted
    "-ffp-contract=off",
    "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
]


def build_library(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB]
    if verbose:
        print(" ".join(cmd))
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is harmless
    noise = "packed-fp32-ops"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
