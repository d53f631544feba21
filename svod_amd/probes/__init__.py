"""Cost probes for gfx950: small stand-alone HIP programs that measure, on the device, what bounds the
attention kernels: the matrix pipe beside the VALU, LDS-fed MFMAs with live data, and where a launch's
workgroups ran and when (``timeline``).  The reference measures its devices the same way before it prices
a config (``tk/src/probe.rs``); here the results are evidence for the kernels' design, kept as text under
``profiles/``.

    python -m svod_amd.probes            build the probes into svod_amd/probes/bin/ and run them (needs a GPU)
    python -m svod_amd.probes --build    build only
    python -m svod_amd.probes.timeline qwen3_attention    (see timeline.py)
    python -m svod_amd.probes.linear_parts                (see linear_parts.py)
"""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "bin")
PROBES = ["issue_probe", "step_probe"]


def build(verbose: bool = False) -> list:
    from .. import build as lib_build

    os.makedirs(BIN, exist_ok=True)
    out = []
    for name in PROBES:
        exe = os.path.join(BIN, name)
        lib_build._run([lib_build.hipcc(), *lib_build.DEVICE_FLAGS, "-O3", "-std=c++17", "-Wno-unused-command-line-argument",
                        "-o", exe, os.path.join(HERE, name + ".hip")], verbose)
        out.append(exe)
    return out


def run() -> None:
    for name in PROBES:
        exe = os.path.join(BIN, name)
        if not os.path.exists(exe):
            raise RuntimeError(f"{exe} is missing: python -m svod_amd.probes --build")
        print(f"==== {name}", flush=True)
        subprocess.run([exe], check=True)
