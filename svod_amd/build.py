"""Builds ``libsvodk_gfx950.so`` in-tree with hipcc, for gfx950 only.

``python -m svod_amd.build`` compiles every source under ``csrc/`` into the library and
then into the code objects under ``co/`` (``--code-objects``: only those).  The
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
SOURCES = ["ops.cpp", "heads_kernel.hip", "attention_kernel.hip", "combine_kernel.hip", "rows_kernel.hip",
           "linear_kernel.hip", "decode_kernel.hip"]

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


# The attention source is compiled once per head size and once for what does not depend on it
# (its SVODK_HEAD macro), side by side: one translation unit of every instantiation takes minutes.
ATTENTION_PARTS = [0, 32, 48, 64, 128, 256]


def build(verbose: bool = False) -> str:
    from concurrent.futures import ThreadPoolExecutor

    cc = hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    jobs = []
    for src in SOURCES:
        stem = os.path.splitext(src)[0]
        parts = [(f"_h{h}", [f"-DSVODK_HEAD={h}"]) for h in ATTENTION_PARTS] if src == "attention_kernel.hip" else [("", [])]
        for suffix, defines in parts:
            obj = os.path.join(objdir, stem + suffix + ".o")
            jobs.append((obj, [cc, "-x", "hip", *DEVICE_FLAGS, *COMMON_FLAGS, *EXTRA_FLAGS.get(src, []), *defines,
                               *os.environ.get("SVODK_CXXFLAGS", "").split(), "-c", os.path.join(CSRC, src), "-o", obj]))
    workers = max(1, min(len(jobs), os.cpu_count() or 1, int(os.environ.get("MAX_JOBS", "8"))))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        list(pool.map(lambda job: _run(job[1], verbose), jobs))
    _run([cc, *DEVICE_FLAGS, "-shared", "-fPIC", "-o", LIB, *[obj for obj, _ in jobs]], verbose)
    return LIB


def build_code_objects(verbose: bool = False) -> str:
    """Writes ``co/*.co`` — the kernels as stand-alone AMDGPU code objects with flat argument
    records (``code_object.py`` says for whom) — and ``co/manifest.json``, after checking each
    kernel against the loader's conditions."""
    import json

    from . import code_object as co

    from concurrent.futures import ThreadPoolExecutor

    cc = hipcc()
    os.makedirs(co.CO_DIR, exist_ok=True)
    table = co.entries()
    jobs = {}
    for name, e in table.items():
        if e["file"] in jobs:
            continue
        path = os.path.join(co.CO_DIR, e["file"])
        # No argument preload here: a loader that writes its own user registers passes the record's address only.
        extra = [f for f in EXTRA_FLAGS.get(e["source"], []) if "kernarg-preload" not in f]
        extra = [f for i, f in enumerate(extra) if not (f == "-mllvm" and (i + 1 == len(extra) or extra[i + 1] == "-mllvm"))]
        head = [f"-DSVODK_HEAD={e['head']}"] if "head" in e else []  # one head size's full family a file
        jobs[e["file"]] = [cc, "-x", "hip", *DEVICE_FLAGS, "--offload-device-only", "--no-gpu-bundle-output",
                           "-DSVODK_CODE_OBJECT", *head, "-O3", "-std=c++17", "-Wall", "-Wno-unused-command-line-argument",
                           *extra, os.path.join(CSRC, e["source"]), "-o", path]
    workers = max(1, min(len(jobs), os.cpu_count() or 1, int(os.environ.get("MAX_JOBS", "8"))))
    with ThreadPoolExecutor(max_workers=workers) as pool:
        list(pool.map(lambda cmd: _run(cmd, verbose), jobs.values()))
    built = {}
    for f in jobs:
        with open(os.path.join(co.CO_DIR, f), "rb") as fh:
            built[f] = fh.read()
    manifest = {"arch": "gfx950", "record": "buffers are 8-byte addresses, scalars 4-byte integers, in this order at "
                                            "natural alignment; *_bits scalars are an f32's bit pattern",
                "kernels": {}}
    for name, e in table.items():
        kd = co.check(built[e["file"]], name, e["params"])
        manifest["kernels"][name] = {**{k: v for k, v in e.items() if k not in ("source", "head")},
                                     "kernarg_size": kd.kernarg_size, "lds_bytes": kd.group_segment_fixed_size}
    for f in built:
        unlisted = set(co.CodeObject.parse(built[f]).kernels()) - set(table)
        if unlisted:
            raise RuntimeError(f"{f}: kernels without a manifest entry: {sorted(unlisted)}")
    with open(os.path.join(co.CO_DIR, "manifest.json"), "w") as f:
        json.dump(manifest, f, indent=1)
    return str(co.CO_DIR)


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
    if "--code-objects" in sys.argv[1:]:
        print(build_code_objects(verbose=True))
    else:
        print(build(verbose=True))
        print(build_code_objects(verbose=True))
