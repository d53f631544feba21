"""Builds ``libsvodk_gfx950.so`` in-tree with hipcc, for gfx950 only.

``python -m svod_amd.build`` compiles every source under ``csrc/``.  The
library is never built implicitly at import: loading fails loudly when it is
missing, so a stale or absent build cannot hide behind another code path.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsvodk_gfx950.so")
SOURCES = ["ops.cpp", "heads_kernel.hip", "attention_kernel.hip", "combine_kernel.hip", "rows_kernel.hip"]

# Packed-FP32 VALU ops are switched off for device code; the host pass of hipcc
# does not know the feature and says so, which is harmless.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                # MFMA results stay in arch VGPRs: the softmax reads them and the rescale writes them
                # every step, and the AGPR form pays a copy each way.
                "-mllvm", "-amdgpu-mfma-vgpr-form"]
# The attention kernel folds MFMA results with max(): without this every operand is first
# quieted by a max(x, x) of its own (32 extra VALU ops a step).  Nothing in that kernel tests
# for NaN, and infinities (the masks) stay honoured.
# The last one keeps an atomic add what the source says (one lane, no wait on the spot): the
# rewrite for wave-uniform operands waits for the answer where the add is issued.
EXTRA_FLAGS = {"attention_kernel.hip": ["-fno-honor-nans", "-mllvm", "-amdgpu-kernarg-preload-count=16",
                                        "-mllvm", "-amdgpu-atomic-optimizer-strategy=None"]}
COMMON_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-command-line-argument"]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def build(verbose: bool = False) -> str:
    cc = hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, os.path.splitext(src)[0] + ".o")
        cmd = [cc, "-x", "hip", *DEVICE_FLAGS, *COMMON_FLAGS, *EXTRA_FLAGS.get(src, []),
               *os.environ.get("SVODK_CXXFLAGS", "").split(), "-c",
               os.path.join(CSRC, src), "-o", obj]
        _run(cmd, verbose)
        objs.append(obj)
    _run([cc, *DEVICE_FLAGS, "-shared", "-fPIC", "-o", LIB, *objs], verbose)
    return LIB


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = ("packed-fp32-ops", "1 warning generated", "warnings generated")
    err = "\n".join(l for l in proc.stderr.splitlines() if l.strip() and not any(n in l for n in noise))
    if proc.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\nfailed with:\n{proc.stderr}")
    if verbose and err:
        print(err, file=sys.stderr)


if __name__ == "__main__":
    print(build(verbose=True))
