"""What the parts of ``linear_kernel`` cost at the Qwen3 projection shape.

    python -m svod_amd.probes.linear_parts [--build]

Builds the library four times into ``bin/`` — as it is, without the fills past the ring's first stages
(``-DSVODK_LINEAR_WITHOUT_FILLS``), without the stores (``-DSVODK_LINEAR_WITHOUT_STORES``) and without both
(the k loop fed from LDS, its barriers and the epilogue's arithmetic) — and times each, in a process of its
own, on x [8,2048,1024] . w [4096,1024]^T plain and with 24 heads of 128 turned; the library GEMM
(``torch.matmul``, hipBLASLt) is timed on the same operands beside them.  The builds with parts left out
compute wrong results: they exist to be timed.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
VARIANTS = [("as it is", "full", []),
            ("without the fills", "nofills", ["-DSVODK_LINEAR_WITHOUT_FILLS"]),
            ("without the stores", "nostores", ["-DSVODK_LINEAR_WITHOUT_STORES"]),
            ("without fills and stores", "loop", ["-DSVODK_LINEAR_WITHOUT_FILLS", "-DSVODK_LINEAR_WITHOUT_STORES"])]


def lib_path(tag: str) -> str:
    return os.path.join(HERE, "bin", f"libsvodk_linear_{tag}.so")


def build(verbose: bool = False) -> list:
    from concurrent.futures import ThreadPoolExecutor

    from .. import build as b

    cc, made = b.hipcc(), []
    # Every object but the GEMM's is the library's own (python -m svod_amd.build leaves them in svod_amd/build).
    objdir = os.path.join(b.HERE, "build")
    others = [os.path.join(objdir, f) for f in sorted(os.listdir(objdir)) if f.endswith(".o") and f != "linear_kernel.o"]
    os.makedirs(os.path.join(HERE, "bin"), exist_ok=True)

    def one(variant):
        _, tag, flags = variant
        obj = os.path.join(HERE, "bin", f"linear_kernel_{tag}.o")
        b._run([cc, "-x", "hip", *b.DEVICE_FLAGS, *b.COMMON_FLAGS, *b.EXTRA_FLAGS.get("linear_kernel.hip", []), *flags,
                "-c", os.path.join(b.CSRC, "linear_kernel.hip"), "-o", obj], verbose)
        b._run([cc, *b.DEVICE_FLAGS, "-shared", "-fPIC", "-o", lib_path(tag), obj, *others], verbose)
        return lib_path(tag)

    with ThreadPoolExecutor(max_workers=4) as pool:
        made = list(pool.map(one, VARIANTS))
    return made


def time_one(lib: str) -> None:
    import torch

    sys.path.insert(0, ROOT)
    import svod_amd

    svod_amd.load_library(None if lib == "library" else lib)
    from svod_amd import Linear, Rotary, workloads as W

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(5)
    b, t, k, h, hkv, d = 8, 2048, 1024, 16, 8, 128
    n = (h + 2 * hkv) * d
    xs = [torch.randn((b, t, k), generator=g, device=dev).to(torch.bfloat16) for _ in range(4)]
    wt = (torch.randn((n, k), generator=g, device=dev) / 32).to(torch.bfloat16)
    cos, sin = W.rope_table(1e6, t, d, dev)
    cos, sin = (a.to(torch.bfloat16).reshape(1, t, 1, d // 2) for a in (cos, sin))
    outs = [torch.empty((b, t, n), dtype=torch.bfloat16, device=dev) for _ in range(4)]

    def best(call):
        for i in range(8):
            call(i)
        torch.cuda.synchronize()
        us = 1e9
        for _ in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(32):
                call(i)
            e1.record()
            torch.cuda.synchronize()
            us = min(us, e0.elapsed_time(e1) * 1000 / 32)
        return "%6.1f us = %4.0f TFLOP/s" % (us, 2.0 * b * t * n * k / us / 1e6)

    if lib == "library":
        flat = [x.view(b * t, k) for x in xs]
        flat_out = [o.view(b * t, n) for o in outs]
        print("%-28s plain %s" % ("torch.matmul (hipBLASLt)", best(lambda i: torch.matmul(flat[i % 4], wt.t(), out=flat_out[i % 4]))),
              flush=True)
        return
    turned = Linear(rope=Rotary(cos, sin, h + hkv, d))
    name = [v[0] for v in VARIANTS if lib_path(v[1]) == lib][0]
    print("%-28s plain %s | turned %s" % (name, best(lambda i: svod_amd.linear(xs[i % 4], wt, Linear(), out=outs[i % 4])),
                                          best(lambda i: svod_amd.linear(xs[i % 4], wt, turned, out=outs[i % 4]))), flush=True)


def main(argv) -> None:
    if "--build" in argv:
        print("\n".join(build(verbose=True)))
        return
    if argv and argv[0] == "--one":
        time_one(argv[1])
        return
    print("linear_kernel at x [8,2048,1024] . w [4096,1024]^T (137.4 GFLOP), operands rotating over 4 sets, best of 4 x 32 calls")
    for lib in [lib_path(v[1]) for v in VARIANTS] + ["library"]:
        if lib != "library" and not os.path.exists(lib):
            raise RuntimeError(f"{lib} is missing: python -m svod_amd.probes.linear_parts --build")
        subprocess.run([sys.executable, "-m", "svod_amd.probes.linear_parts", "--one", lib], check=True, timeout=300, cwd=ROOT)


if __name__ == "__main__":
    main(sys.argv[1:])
