"""Where and when the workgroups of one attention launch ran.

    python -m svod_amd.probes.timeline [--build] [bge_m3|qwen3_attention|whisper|long] [--no-row-order] [--raw=FILE.npy]

Builds ``bin/libsvodk_timeline.so``, the library with ``-DSVODK_TIMELINE`` (thread 0 of every workgroup of
``flash_fwd_kernel`` stamps the 100 MHz clock at entry, first fills issued, first barrier, last computed
step, last step and stores landed, and notes its XCD, shader engine and CU), runs one call of a ``bench.py`` workload after
warm-up and prints: the launch's span against the sum of the workgroups' own times, their phases, the
time per key block, how many workgroups are resident over time, the gaps between one workgroup's end and
the next one's start on a CU, each XCD's share of the time and its last end, and how each XCD deals
workgroups to its shader engines.  The stamps cost
time themselves (a launch takes about a quarter longer): proportions count, not microseconds.
"""
from __future__ import annotations

import ctypes
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
LIB = os.path.join(HERE, "bin", "libsvodk_timeline.so")


def build(verbose: bool = False) -> str:
    from concurrent.futures import ThreadPoolExecutor

    from .. import build as b

    objdir = os.path.join(HERE, "bin", "timeline_objs")
    os.makedirs(objdir, exist_ok=True)
    cc, jobs = b.hipcc(), []
    for src in b.SOURCES:
        stem = os.path.splitext(src)[0]
        parts = [(f"_h{h}", [f"-DSVODK_HEAD={h}"]) for h in b.ATTENTION_PARTS] if src == "attention_kernel.hip" else [("", [])]
        for suffix, defines in parts:
            obj = os.path.join(objdir, stem + suffix + ".o")
            jobs.append((obj, [cc, "-x", "hip", *b.DEVICE_FLAGS, *b.COMMON_FLAGS, *b.EXTRA_FLAGS.get(src, []), *defines,
                               "-DSVODK_TIMELINE", "-c", os.path.join(b.CSRC, src), "-o", obj]))
    with ThreadPoolExecutor(max_workers=8) as pool:
        list(pool.map(lambda job: b._run(job[1], verbose), jobs))
    b._run([cc, *b.DEVICE_FLAGS, "-shared", "-fPIC", "-o", LIB, *[obj for obj, _ in jobs]], verbose)
    return LIB


def main(argv) -> None:
    if "--build" in argv:
        print(build(verbose=True))
        return
    import numpy as np
    import torch

    sys.path.insert(0, ROOT)
    import svod_amd

    if not os.path.exists(LIB):
        raise RuntimeError(f"{LIB} is missing: python -m svod_amd.probes.timeline --build")
    lib = svod_amd.load_library(LIB)
    import bench

    names = [a for a in argv if not a.startswith("--")]
    name = names[0] if names else "qwen3_attention"

    class Args:
        layers, calls = 4, 4

    dev = torch.device("cuda:0")
    wl = bench.build_workload(name, Args, dev, row_order="--no-row-order" not in argv)
    head = 128 if name.startswith("qwen3") else 64
    point = getattr(lib, f"svodk_debug_timeline_h{head}")
    point.argtypes, point.restype = [ctypes.c_void_p], ctypes.c_int
    buf = torch.zeros((1 << 16) * 8, dtype=torch.int64, device=dev)
    for _ in range(3):
        wl.step()
    for c in wl.extra_calls:
        c()
    for _ in range(6):
        wl.calls[1]()
    torch.cuda.synchronize()
    assert point(buf.data_ptr()) == 0
    wl.calls[0]()
    torch.cuda.synchronize()
    point(None)
    t = buf.cpu().numpy().astype(np.uint64).reshape(-1, 8)
    t = t[t[:, 0] != 0]
    raw = [a.split("=", 1)[1] for a in argv if a.startswith("--raw=")]
    if raw:
        np.save(raw[0], t)  # a row a workgroup, in launch order: the five stamps, the hardware id, blocks << 32
    t0 = np.int64(t[:, 0].min())
    start, first, loop_end, idle_end, end = ((t[:, c].astype(np.int64) - t0) * 0.01 for c in range(5))  # us
    hw, xcc = t[:, 5] & 0xffffffff, (t[:, 5] >> 32) & 0xf
    cu, se = (hw >> 8) & 0xf, (hw >> 13) & 0x7
    key = (xcc * 1000 + se * 32 + cu).astype(np.int64)
    blocks = np.maximum((t[:, 6] >> 32).astype(np.int64), 1)
    span, dur = end.max(), end - start
    cus = np.unique(key)
    most = max(int(((start <= x) & (end > x)).sum()) for x in np.arange(0, span, 1.0))
    per_cu = max(1, int(round(most / len(cus))))
    slots = per_cu * len(cus)
    print(f"{wl.text}")
    print(f"workgroups {len(t)}, compute units {len(cus)}, resident workgroups a CU {per_cu}")
    print(f"span {span:.1f} us; the workgroups' own times sum to {dur.sum():.0f} us = {dur.sum() / slots:.1f} us a slot "
          f"({100 * dur.sum() / slots / span:.0f} % of the span)")
    pct = lambda x: "mean %.2f  p50 %.2f  p90 %.2f" % (x.mean(), *np.percentile(x, [50, 90]))
    fills_out = (t[:, 7].astype(np.int64) - t0) * 0.01
    print("entry -> first fills out    ", pct(fills_out - start))
    print("entry -> first barrier      ", pct(first - start))
    print("first barrier -> last step  ", pct(idle_end - first), " per key block", pct((idle_end - first) / blocks))
    print("last step -> stores landed  ", pct(end - idle_end))
    coef, *_ = np.linalg.lstsq(np.stack([np.ones(len(t)), blocks.astype(float)], 1), dur, rcond=None)
    print("a workgroup's time ~= %.2f + %.3f us x key blocks" % tuple(coef))
    grid = np.arange(0, span, max(2.0, span / 40))
    print("resident workgroups over time:", [int(((start <= x) & (end > x)).sum()) for x in grid])
    gaps = []
    for k in cus:
        events = sorted([(start[i], 1) for i in np.nonzero(key == k)[0]] + [(end[i], 0) for i in np.nonzero(key == k)[0]])
        free = []
        for when, is_start in events:
            if not is_start:
                free.append(when)
            elif free:
                gaps.append(when - free.pop(0))
    gaps = np.array(gaps) if gaps else np.zeros(1)
    print("gap between a workgroup's end and the next start on its CU:", pct(gaps), " max %.1f;" % gaps.max(),
          "gaps sum to %.0f %% of the slots' time, the ragged end to %.0f %%" %
          (100 * gaps.sum() / (slots * span), 100 * (slots * span - dur.sum() - gaps.sum()) / (slots * span)))
    print("per XCD: the workgroups' own times sum to", [int(dur[xcc == x].sum()) for x in range(8)], "us; last end",
          [round(float(end[xcc == x].max()), 1) for x in range(8)])
    print("per XCD: entry -> first barrier, mean", [round(float((first - start)[xcc == x].mean()), 2) for x in range(8)])
    ends = np.array([end[key == k].max() for k in cus])
    print("a CU's last end: min %.1f  p50 %.1f  max %.1f" % (ends.min(), np.median(ends), ends.max()))
    order = np.argsort(t[:, 0], kind="stable")
    x0 = np.nonzero(xcc == 0)[0]
    print("XCD 0 deals its workgroups, in launch order, to shader engines", se[x0][:16].tolist(), "...")
    print("XCD of workgroup i is i % 8 for", "%.0f %%" % (100 * np.mean(xcc == np.arange(len(t)) % 8)) if len(t) == int(t.shape[0]) else "?",
          "of the workgroups")


if __name__ == "__main__":
    main(sys.argv[1:])
