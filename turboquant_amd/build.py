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
# (the matrix-core page kernel is instantiated by one file per head size, so that they compile side by side)
SOURCES = ["tq_decode_mfma_d128.hip", "tq_decode_mfma_d128_f16.hip", "tq_decode_mfma_d64.hip", "tq_decode_mfma_d64_f16.hip",
           "tq_decode_mfma_d256.hip", "tq_quantize_mfma.hip", "tq_decode_wide.hip",
           "tq_quantize.hip", "tq_score.hip", "tq_decode.hip", "tq_decode_mfma.hip", "tq_probe.hip"]

# packed-fp32 instructions stay off: some of their forms have produced wrong
# results on this hardware pool
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # no implicit a*b+c fusion: the quantisers mirror separately rounded torch ops;
    # the kernels call fmaf() explicitly wherever a fused multiply-add is wanted
    "-ffp-contract=off",
    "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
    # the LDS-direct loads name m0 in their clobber lists, which the compiler reports as a reserved register
    "-Wno-inline-asm",
]


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass warns that it does not know the packed-fp32 feature; that is harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    return res.returncode, err


def build_library(verbose: bool = False) -> str:
    """Compile every source to an object file (in parallel: the files are independent translation units)
    and link them into libtq_hip.so."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    # TQ_EXTRA_HIPCC_FLAGS: extra compile flags, e.g. -DTQ_STAMPS for the page kernel's phase time stamps
    compile_flags = [f for f in FLAGS if f != "-shared"] + os.environ.get("TQ_EXTRA_HIPCC_FLAGS", "").split()
    jobs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        jobs.append((obj, [hipcc] + compile_flags + ["-c", os.path.join(CSRC, src), "-o", obj]))
    if verbose:
        for _, cmd in jobs:
            print(" ".join(cmd))
    with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1)) as pool:
        results = list(pool.map(lambda j: _run(j[1]), jobs))
    for (obj, _), (rc, err) in zip(jobs, results):
        if rc != 0:
            raise RuntimeError(f"hipcc failed ({rc}) for {obj}:\n{err}")
        if verbose and err.strip():
            print(err, file=sys.stderr)
    link = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc"] + [obj for obj, _ in jobs] + ["-o", LIB]
    if verbose:
        print(" ".join(link))
    rc, err = _run(link)
    if rc != 0:
        raise RuntimeError(f"hipcc link failed ({rc}):\n{err}")
    return LIB


if __name__ == "__main__":
    print(build_library(verbose=True))
