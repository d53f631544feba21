#!/usr/bin/env python3
"""Benchmark of the tk flash-attention forward path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints ONE JSON line.  The default workload is the configuration the headline
metric is quoted on: BGE-M3 / XLM-R-large encoder self-attention, bf16, batch 32,
16 heads, head_dim 64, S 512, key padding U[64, 512], one model forward's worth
of calls (24 layers, 24 independent seeded Q/K/V sets).  A "step" is that forward:
24 attention calls enqueued back to back, inputs resident in HBM.

``value`` is TFLOP/s over the FLOPs of visible (query, key) pairs; the reference's
own convention (4·b·h·t·tk·d, tk/examples/tk_bench.rs:277) is reported beside it.
The ``roofline`` object prices the attention kernel against the bf16 dense MFMA
peak; ``cpu_baseline`` times the CPU restatement of the reference's graph path on
a bounded sample of the same inputs, on this box's host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBS = 8000.0
ROOT = os.path.dirname(os.path.abspath(__file__))
# The workloads a default run times after the headline one, a few steps each, so that one run
# carries every figure the targets are set on.
OTHERS = ["bge_m3_bool", "qwen3_attention", "qwen3_prologue", "qwen3_add_rms_norm", "whisper", "long", "whisper_decode",
          "qwen3_projection"]


def hbm_traffic(workload):
    """HBM bytes per launch of the workload's dominant kernel, from profiles/traffic.json: rocprofv3
    --pmc FETCH_SIZE and WRITE_SIZE runs of this file, each scaled by what the counter reads for a 256 MiB
    device copy (the summaries under profiles/ give the commands).  Counters cannot be read from inside a
    timed run; a workload that has not been profiled reports null."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get("bytes_per_launch", {}).get(workload)
    except (OSError, ValueError):
        return None


def device_clock_mhz():
    """The device's peak engine clock in MHz, asked of the HIP runtime torch has loaded
    (hipDeviceGetAttribute, hipDeviceAttributeClockRate), or a string that says why there is none."""
    import ctypes

    try:
        hip = ctypes.CDLL("libamdhip64.so")
        khz = ctypes.c_int(0)
        rc = hip.hipDeviceGetAttribute(ctypes.byref(khz), ctypes.c_int(5), ctypes.c_int(0))  # 5: ClockRate, kHz
        if rc != 0 or khz.value <= 0:
            return "unavailable: hipDeviceGetAttribute(ClockRate) returned %d" % rc
        return khz.value // 1000
    except OSError as e:
        return "unavailable: %s" % e


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="bge_m3",
                    choices=["bge_m3", "bge_m3_bool", "qwen3_attention", "qwen3_prologue", "qwen3_add_rms_norm",
                             "whisper", "whisper_decode", "long", "qwen3_projection", "qwen3_projection_plain", "hbm_copy"],
                    help="hbm_copy is a plain 256 MiB device copy: the known-size kernel the HBM counters "
                         "(FETCH_SIZE, WRITE_SIZE) are calibrated on")
    ap.add_argument("--layers", type=int, default=24, help="calls per step for the bge_m3 workloads")
    ap.add_argument("--calls", type=int, default=16,
                    help="calls per step for the other workloads, rotating over 4 copies of the operands so that "
                         "none is served from the Infinity Cache")
    ap.add_argument("--no-graph", action="store_true", help="enqueue eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-row-order", action="store_true",
                    help="bge_m3, bge_m3_bool, qwen3_attention: take the batch rows as they come instead of ordering them by "
                         "length once per step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="rough budget of the CPU baseline sample")
    ap.add_argument("--no-others", action="store_true",
                    help="the default workload only: without the shorter runs of the other configurations that a "
                         "default run appends under \"others\"")
    ap.add_argument("--other-steps", type=int, default=4, help="timed steps of each workload under \"others\"")
    return ap.parse_args()


class Workload:
    """A step of one workload: closures that launch on the current stream, and what a launch is worth."""

    def __init__(self):
        self.calls, self.extra_calls = [], []  # extra: launches of a step that are not calls of the op measured
        self.flops_vis = self.flops_nom = 0.0
        self.bytes_min = 0
        self.kernel_name, self.bound, self.text = "", "mfma", ""
        self.cpu_sample = None
        self.keep = []  # what the closures use

    def step(self):
        for c in self.extra_calls:
            c()
        for c in self.calls:
            c()


def build_workload(name, args, dev, row_order=True):
    import torch

    import svod_amd
    from svod_amd import Attn, KeyMask, Qkv, workloads as W

    wl = Workload()
    calls = wl.calls
    if name in ("bge_m3", "bge_m3_bool"):
        sets = [W.config2(layer=l, device=dev) for l in range(args.layers)]
        # The lengths belong to the batch, not to a layer (every set has the same ones): as a model would,
        # the step orders the batch rows by length once (one small launch, inside the timed region) and
        # hands the order to its 24 layer calls.  --no-row-order runs the rows as they come.
        order = None
        if row_order:
            order = torch.empty(sets[0].key_lens.shape, dtype=torch.int32, device=dev)
            keys0 = sets[0].key_lens if name == "bge_m3" else sets[0].key_mask()
            wl.extra_calls.append(lambda: svod_amd.order_rows(keys0, out=order))
        for w in sets:
            keys = KeyMask.lens(w.key_lens) if name == "bge_m3" else KeyMask.bool(w.key_mask())
            out = torch.empty_like(w.q)
            calls.append((lambda w=w, keys=keys, out=out: svod_amd.attention(
                w.q, w.k, w.v, Attn(keys=keys, scale=w.scale, row_order=order), out=out)))
        w0 = sets[0]
        wl.flops_vis, wl.flops_nom, wl.bytes_min = w0.visible_flops(), w0.nominal_flops(), w0.min_bytes()
        wl.text = "BGE-M3 encoder self-attention bf16 B32 H16 D64 S512 key-padding U[64,512], %d layer calls/step%s%s" % (
            args.layers, " (KeyMask::Bool)" if name == "bge_m3_bool" else " (KeyMask::Lens)",
            ", batch rows ordered by length once per step (svodk_order_rows, in the timed region)" if order is not None else "")
        wl.cpu_sample = ("attention", w0)
        wl.kernel_name = "flash_fwd_kernel<64>"
    elif name == "hbm_copy":
        srcs = [torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(2)]
        dsts = [torch.empty_like(x) for x in srcs]
        for i in range(args.calls):
            calls.append(lambda i=i: dsts[i % 2].copy_(srcs[i % 2]))
        wl.bytes_min = 2 * srcs[0].numel()
        wl.text = "plain device copy of 256 MiB (torch copy_), counter calibration"
        wl.kernel_name, wl.bound = "torch elementwise copy", "hbm"
    elif name == "qwen3_prologue":
        p = W.config3_prologue(device=dev)
        opts = Qkv(p.heads, p.kv_heads, p.head_dim, p.q_w, p.k_w, p.eps, (p.cos, p.sin))
        ins = [p.qkv] + [p.qkv.clone() for _ in range(3)]
        outs = [tuple(torch.empty((8, 2048, n, 128), dtype=torch.bfloat16, device=dev) for n in (16, 8, 8))
                for _ in range(4)]
        for i in range(args.calls):
            calls.append(lambda i=i: svod_amd.heads(ins[i % 4], opts, out=outs[i % 4]))
        wl.bytes_min = p.min_bytes()
        wl.text = "Qwen3-Embedding prologue bf16 qkv[8,2048,4096] -> q,k,v (RMSNorm eps 1e-6 + RoPE theta 1e6)"
        wl.cpu_sample = ("heads", p)
        wl.kernel_name, wl.bound = "heads_kernel<128>", "hbm"
    elif name in ("qwen3_projection", "qwen3_projection_plain"):
        # The fused q/k/v projection at Qwen3-Embedding's shape with the rope applied in the GEMM's store (what a
        # model without QK norms runs, tk/src/ops/linear.rs:47-58): x [8,2048,1024] . w [4096,1024]^T, 16 + 8 heads
        # of 128 turned.  The plain form is the same GEMM without the turn.
        from svod_amd import Linear, Rotary
        g = torch.Generator(device=dev).manual_seed(0x5EED0038)
        b, t, k, h, hkv, d = 8, 2048, 1024, 16, 8, 128
        n = (h + 2 * hkv) * d
        xs = [torch.randn((b, t, k), generator=g, device=dev).to(torch.bfloat16) for _ in range(4)]
        wt = (torch.randn((n, k), generator=g, device=dev) / 32).to(torch.bfloat16)
        cos, sin = W.rope_table(1e6, t, d, dev)
        cos, sin = (a.to(torch.bfloat16).reshape(1, t, 1, d // 2) for a in (cos, sin))
        outs = [torch.empty((b, t, n), dtype=torch.bfloat16, device=dev) for _ in range(4)]
        opts = Linear(rope=Rotary(cos, sin, h + hkv, d)) if name == "qwen3_projection" else Linear()
        for i in range(args.calls):
            calls.append(lambda i=i: svod_amd.linear(xs[i % 4], wt, opts, out=outs[i % 4]))
        wl.flops_vis = wl.flops_nom = 2.0 * b * t * n * k
        wl.bytes_min = (xs[0].numel() + wt.numel() + outs[0].numel()) * 2
        wl.text = ("fused q/k/v projection bf16 x[8,2048,1024] . w[4096,1024]^T" +
                   (", 24 heads of 128 turned in the store (rope theta 1e6)" if name == "qwen3_projection" else ", no turn"))
        wl.kernel_name = "linear_kernel<rope 128>" if name == "qwen3_projection" else "linear_kernel"
        wl.cpu_sample = ("linear", (xs[0], wt, cos, sin, h + hkv, d))
    elif name == "whisper_decode":
        # One decoder step of Whisper-large-v3's cross-attention (model/src/whisper/decoder.rs:441-477): a query
        # per lane against the 1500 encoder keys of its layer, read from a cache that holds every layer's heads.
        from svod_amd import Cache
        g = torch.Generator(device=dev).manual_seed(0x5EED0040)
        b, tk, h, d, layers = 16, 1500, 20, 64, 32
        k_cache = torch.randn((b, tk, layers * h, d), generator=g, device=dev).to(torch.bfloat16)
        v_cache = torch.randn((b, tk, layers * h, d), generator=g, device=dev).to(torch.bfloat16)
        qs = [torch.randn((b, 1, h, d), generator=g, device=dev).to(torch.bfloat16) for _ in range(layers)]
        outs = [torch.empty_like(qs[0]) for _ in range(layers)]
        lens = torch.full((b,), tk, dtype=torch.int32, device=dev)
        ws = torch.empty(8 * b * h * (d + 2) * 4, dtype=torch.uint8, device=dev)
        for layer in range(layers):
            calls.append(lambda layer=layer: svod_amd.attention(
                qs[layer], k_cache, v_cache, Attn(keys=KeyMask.lens(lens), cache=Cache(layer * h, h)), out=outs[layer],
                workspace=ws))
        wl.bytes_min = 2 * b * tk * h * d * 2 + 2 * b * h * d * 2  # the layer's K and V heads read once, q and o
        wl.text = ("Whisper-large-v3 decoder step, cross-attention bf16 B16 T1 H20 D64 over 1500 cached keys, "
                   "32 layer calls/step on one cache [16,1500,640,64] (splits chosen by the library)")
        wl.kernel_name, wl.bound = "decode_kernel<64, split> + combine_kernel<64>", "hbm"
    elif name == "qwen3_add_rms_norm":
        # The residual add + RMSNorm between Qwen3-Embedding's layers: hidden size 16 heads x 128 = 2048.
        g = torch.Generator(device=dev).manual_seed(0x5EED0030)
        shape = (8, 2048, 2048)
        xs = [torch.randn(shape, generator=g, device=dev).to(torch.bfloat16) for _ in range(4)]
        rs = [torch.randn(shape, generator=g, device=dev).to(torch.bfloat16) for _ in range(4)]
        wn = (0.8 + 0.4 * torch.rand(2048, generator=g, device=dev)).to(torch.bfloat16)
        outs = [(torch.empty_like(xs[0]), torch.empty_like(xs[0])) for _ in range(4)]
        for i in range(args.calls):
            calls.append(lambda i=i: svod_amd.add_rms_norm(xs[i % 4], rs[i % 4], wn, 1e-6, out=outs[i % 4]))
        wl.bytes_min = 4 * xs[0].numel() * 2 + 2 * 2048  # x and residual read, sum and out written, the weight
        wl.text = "Qwen3-Embedding residual add + RMSNorm bf16 x,residual [8,2048,2048] -> sum, out (eps 1e-6)"
        wl.cpu_sample = ("norm", (xs[0], rs[0], wn))
        wl.kernel_name, wl.bound = "rows_kernel<4, rms, residual>", "hbm"
    else:
        if name == "qwen3_attention":
            p = W.config3_prologue(device=dev)
            q, k, v = svod_amd.heads(p.qkv, Qkv(p.heads, p.kv_heads, p.head_dim, p.q_w, p.k_w, p.eps, (p.cos, p.sin)))
            w = W.config3_attention(q, k, v)
            wl.text = "Qwen3-Embedding causal GQA attention bf16 B8 S2048 Hq16 Hkv8 D128, right padding U[512,2048]"
            wl.kernel_name = "flash_fwd_kernel<128, causal>"
        elif name == "whisper":
            w = W.config4(device=dev)
            wl.text = "Whisper-large-v3 encoder attention bf16 B16 H20 D64 S1500, no mask"
            wl.kernel_name = "flash_fwd_kernel<64>"
        else:
            w = W.config5(device=dev)
            wl.text = "long-context pair attention bf16 B2 H16 D64 S8192, lens {8192, 5000}"
            wl.kernel_name = "flash_fwd_kernel<64>"
        keys = KeyMask.lens(w.key_lens) if w.key_lens is not None else KeyMask.none()
        ins = [(w.q, w.k, w.v)] + [(w.q.clone(), w.k.clone(), w.v.clone()) for _ in range(3)]
        outs = [torch.empty_like(w.q) for _ in range(4)]
        # Ragged batches are ordered by length once per step, like the bge_m3 rows above (--no-row-order: as given).
        order = None
        if row_order and name == "qwen3_attention":
            order = torch.empty(w.key_lens.shape, dtype=torch.int32, device=dev)
            wl.extra_calls.append(lambda: svod_amd.order_rows(w.key_lens, out=order))
            wl.text += ", batch rows ordered by length once per step"
        opts = Attn(causal=w.causal, keys=keys, scale=w.scale, row_order=order)
        for i in range(args.calls):
            calls.append(lambda i=i: svod_amd.attention(*ins[i % 4], opts, out=outs[i % 4]))
        wl.flops_vis, wl.flops_nom, wl.bytes_min = w.visible_flops(), w.nominal_flops(), w.min_bytes()
        wl.cpu_sample = ("attention", w)
    return wl


def measure(wl, steps, warmup, use_graph=True, spread=True, warm=True):
    """Times `steps` steps of the workload between synchronisations, after `warmup` untimed ones and a
    clock warm-up.  Every launch goes to torch's current stream, which is also where the events are
    recorded.  Returns ms per step, the average launch duration and the extras asked for."""
    import torch

    step = wl.step
    # ---- warm-up (also loads the code objects and sets kernel attributes), then capture.
    for _ in range(max(1, warmup)):
        step()
    torch.cuda.synchronize()
    graph = None
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        graph.replay()
        torch.cuda.synchronize()
    run = graph.replay if graph is not None else step

    # Clock warm-up: back-to-back steps until the windowed minimum stops improving
    # (after the reference tuner, tk/src/tune.rs:97-131).
    best, t_end = float("inf"), time.time() + 0.4
    while True:
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            run()
        e1.record()
        e1.synchronize()
        ms = e0.elapsed_time(e1) / 3
        if ms < 0.95 * best:
            best = ms
        elif time.time() > t_end:
            break
        best = min(best, ms)

    # ---- the timed region: exactly K steps between synchronisations.
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    wall0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        run()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - wall0) * 1e3
    gpu_ms = e0.elapsed_time(e1)
    res = {"ms_per_step": max(wall_ms, gpu_ms) / steps,
           "kernel_us": gpu_ms * 1e3 / (len(wl.calls) * steps),  # average launch duration over the timed region (HIP events)
           "launch": "hip graph replay" if graph is not None else "eager"}

    if spread:
        # Five more rounds of K steps for the spread (min and median, after the reference tuner's
        # reporting, runtime/src/benchmark.rs:13-52); the headline stays the timed region above.
        rounds = []
        for _ in range(5):
            r0, r1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            r0.record()
            for _ in range(steps):
                run()
            r1.record()
            r1.synchronize()
            rounds.append(r0.elapsed_time(r1) / steps)
        rounds.sort()
        res["rounds"] = rounds
    if warm:
        # The same call back to back on one operand set: operands warm in the Infinity Cache (the
        # reference's tuner times cold, its probes warm; both are reported, the headline is cold).
        for c in wl.extra_calls:
            c()
        n_warm = max(len(wl.calls) * steps // 4, 8)
        for _ in range(4):
            wl.calls[0]()
        w0, w1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        w0.record()
        for _ in range(n_warm):
            wl.calls[0]()
        w1.record()
        w1.synchronize()
        res["warm_us"] = w0.elapsed_time(w1) * 1e3 / n_warm
    return res


def roofline(name, wl, kernel_us):
    if wl.bound == "mfma":
        achieved = wl.flops_vis / (kernel_us * 1e-6) / 1e12
        return {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": hbm_traffic(name),
                "traffic_unit": "bytes per launch", "kernel": wl.kernel_name,
                "kernel_us": round(kernel_us, 3), "flops_per_launch_visible": wl.flops_vis,
                "flops_per_launch_nominal": wl.flops_nom,
                "nominal_tflops": round(wl.flops_nom / (kernel_us * 1e-6) / 1e12, 2),
                "hbm_gbs_at_min_bytes": round(wl.bytes_min / (kernel_us * 1e-6) / 1e9, 1)}
    achieved = wl.bytes_min / (kernel_us * 1e-6) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": hbm_traffic(name),
            "traffic_unit": "bytes per launch", "kernel": wl.kernel_name,
            "kernel_us": round(kernel_us, 3), "bytes_per_launch": wl.bytes_min}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (every (batch, head, query tile) block is "
              "independent, so the op shards over batch and heads without exchange); run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)

    import torch

    import svod_amd

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(2)
    svod_amd.load_library()
    if not svod_amd.supported():
        print("the current device is not a gfx950 this library has kernels for", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(0)

    name = args.workload
    wl = build_workload(name, args, dev, row_order=not args.no_row_order)
    m = measure(wl, args.steps, args.warmup, use_graph=not args.no_graph)
    ms_per_step, kernel_us, rounds = m["ms_per_step"], m["kernel_us"], m["rounds"]
    roof = roofline(name, wl, kernel_us)
    calls = wl.calls
    if wl.bound == "mfma":
        value = wl.flops_vis * len(calls) / (ms_per_step * 1e-3) / 1e12
        metric, unit = "flash-attn fwd TFLOP/s (visible-pair FLOPs) on 1 MI355X", "TFLOP/s"
        if name.startswith("qwen3_projection"):
            metric = "fused projection GEMM TFLOP/s on 1 MI355X"
    else:
        value = wl.bytes_min * len(calls) / (ms_per_step * 1e-3) / 1e9
        metric = {"qwen3_add_rms_norm": "row norm GB/s on 1 MI355X",
                  "whisper_decode": "decoder-step attention GB/s of K and V on 1 MI355X"}.get(
                      name, "attention prologue GB/s on 1 MI355X")
        unit = "GB/s"

    config = {"workload": wl.text, "calls_per_step": len(calls), "ms_per_call": round(ms_per_step / len(calls), 5),
              "launch": m["launch"],
              "ms_per_step_min": round(rounds[0], 5), "ms_per_step_median": round(rounds[2], 5),
              "us_per_call_warm": round(m["warm_us"], 2),
              "operands": "cold: the calls of a step rotate over operand sets larger than the 256 MB Infinity Cache "
                          "(us_per_call_warm: one set back to back, eager launches)",
              "device": props.name or props.gcnArchName, "compute_units": props.multi_processor_count,
              "clock_mhz": device_clock_mhz(),
              "clock_note": "peak engine clock the runtime reports; the roofline peaks are MI355X's published ones "
                            "(2.5 PFLOP/s dense bf16 at 2.4 GHz, 8 TB/s)"}

    # ---- CPU baseline: the oracle's restatement of the reference graph path, bounded sample.
    cpu = None
    if not args.no_cpu_baseline and wl.cpu_sample is not None:
        cpu = cpu_baseline(wl.cpu_sample, args.cpu_seconds, wl.bound)

    others = None
    if name == "bge_m3" and not args.no_others:
        # The same calls with the batch rows as the caller gave them (no svodk_order_rows, no row_order): the
        # figure of the op exactly as the reference has it, beside the headline.
        if not args.no_row_order:
            plain = build_workload(name, args, dev, row_order=False)
            pm = measure(plain, max(2, args.steps // 4), 1, use_graph=not args.no_graph, spread=False, warm=False)
            config["us_per_call_rows_as_given"] = round(pm["kernel_us"], 3)
            config["frac_rows_as_given"] = roofline(name, plain, pm["kernel_us"])["frac"]
            del plain
        del wl
        torch.cuda.empty_cache()
        others = []
        for other in OTHERS:
            ow = build_workload(other, args, dev)
            om = measure(ow, args.other_steps, 2, use_graph=not args.no_graph, spread=False, warm=False)
            r = roofline(other, ow, om["kernel_us"])
            entry = {"workload": ow.text, "name": other, "calls_per_step": len(ow.calls), "steps": args.other_steps,
                     "kernel": r["kernel"], "kernel_us": r["kernel_us"], "bound": r["bound"],
                     "achieved": r["achieved"], "unit": r["unit"], "peak": r["peak"], "frac": r["frac"],
                     "traffic": r["traffic"]}
            if other == "qwen3_prologue" and not args.no_cpu_baseline:
                # ms/call against the host CPU for the prologue too: a short bounded sample of its graph path.
                entry["cpu_baseline"] = cpu_baseline(ow.cpu_sample, min(args.cpu_seconds, 3.0), ow.bound)
            others.append(entry)
            del ow
            torch.cuda.empty_cache()

    line = {
        "metric": metric, "value": round(value, 3), "unit": unit, "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": config, "roofline": roof, "cpu_baseline": cpu,
    }
    if others is not None:
        line["others"] = others
    print(json.dumps(line))


def cpu_baseline(sample, seconds, bound):
    """Time the oracle (a port of the reference's CPU graph path) on a bounded sample."""
    import numpy as np

    import oracle

    kind, w = sample
    cores = min(os.cpu_count() or 1, 16)
    if kind == "norm":
        rows = 4096
        x, r = (a.reshape(-1, a.shape[-1])[:rows].float().cpu().numpy() for a in w[:2])
        wn = w[2].float().cpu().numpy()
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < min(seconds, 5.0):
            oracle.norm_f32(oracle.RMS, x, wn, residual=r, eps=1e-6)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        nbytes = 4 * x.size * 2
        return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{rows} rows of one call (x, residual [{rows},2048]), f32 restatement of the graph path, "
                          f"scalar C, {reps} reps"}
    if kind == "linear":
        x, wt, cos, sin, heads, d = w
        rows = 4
        xs = x[:1, :rows].float().cpu().numpy()
        wn = wt.float().cpu().numpy()
        rope = (cos[0, :rows, 0].float().cpu().numpy(), sin[0, :rows, 0].float().cpu().numpy(), heads, d)
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < min(seconds, 5.0):
            oracle.linear_kernel(xs, wn, None, rope)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        return {"value": round(2.0 * rows * wn.shape[0] * wn.shape[1] / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
                "kind": "port", "sample": f"{rows} rows of batch 0, f32 restatement of the kernel's arithmetic, scalar C, {reps} reps"}
    if kind == "heads":
        rows = 256
        qkv = w.qkv[:1, :rows].float().cpu().numpy()
        prob = oracle.HeadsProblem(qkv, w.heads, w.kv_heads, w.head_dim, w.q_w.float().cpu().numpy(),
                                   w.k_w.float().cpu().numpy(), w.eps, w.cos[0, :rows, 0].float().cpu().numpy(),
                                   w.sin[0, :rows, 0].float().cpu().numpy())
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < min(seconds, 5.0):
            oracle.heads_graph(prob)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        nbytes = 2 * qkv.size * 2
        return {"value": round(nbytes / dt / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{rows} rows of batch 0 (qkv [1,{rows},4096]), graph restatement, scalar C, {reps} reps"}
    b, t, tk, h, hkv, d = w.dims
    # Size the sample from a probe of one batch row.
    def problem(nb):
        lens = None if w.key_lens is None else w.key_lens[:nb].cpu().numpy()
        return oracle.AttnProblem(w.q[:nb].float().cpu().numpy(), w.k[:nb].float().cpu().numpy(),
                                  w.v[:nb].float().cpu().numpy(), causal=w.causal, key_lens=lens, scale=w.scale)
    pairs = lambda nb: oracle.visible_pairs(nb, t, tk, w.causal, None if w.key_lens is None else w.key_lens[:nb].cpu().numpy())
    if 4.0 * b * h * t * tk * d > 2e11:  # a long sequence: sample heads of one batch row instead
        sub = W_slice_heads(w, 1, min(h, cores))
        prob, npairs, nheads, what = sub
        t0 = time.perf_counter()
        oracle.attention_graph(prob, threads=cores)
        dt = time.perf_counter() - t0
        flops = 4.0 * d * nheads * npairs
        return {"value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port", "sample": what}
    t0 = time.perf_counter()
    oracle.attention_graph(problem(1), threads=cores)
    probe = time.perf_counter() - t0
    nb = int(max(1, min(b, seconds / max(probe, 1e-3))))
    prob = problem(nb)
    t0 = time.perf_counter()
    oracle.attention_graph(prob, threads=cores)
    dt = time.perf_counter() - t0
    flops = 4.0 * d * h * pairs(nb)
    return {"value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": f"batch rows 0..{nb - 1} of one call ({nb}x{h} (batch, head) slices, visible-pair FLOPs), "
                      f"C restatement of the reference graph path, {cores} threads, {dt:.2f} s"}


def W_slice_heads(w, nb, nh):
    import oracle

    b, t, tk, h, hkv, d = w.dims
    group = h // hkv
    nh = max(group, (nh // group) * group)
    lens = None if w.key_lens is None else w.key_lens[:nb].cpu().numpy()
    prob = oracle.AttnProblem(w.q[:nb, :, :nh].float().cpu().numpy(), w.k[:nb, :, :nh // group].float().cpu().numpy(),
                              w.v[:nb, :, :nh // group].float().cpu().numpy(), causal=w.causal, key_lens=lens,
                              scale=w.scale)
    npairs = oracle.visible_pairs(nb, t, tk, w.causal, lens)
    what = (f"heads 0..{nh - 1} of batch row 0 ({nh} (batch, head) slices, visible-pair FLOPs), "
            f"C restatement of the reference graph path")
    return prob, npairs, nh, what


if __name__ == "__main__":
    main()
