"""The launch path as its callers use it: captured into a HIP graph and replayed (what a plan replay of
the reference does with its kernels, runtime/src/execution_plan.rs), and from several host threads at once
(device/src/device.rs:33-36: a program is "stateless and reentrant from the host perspective").  Every
replay and every thread must give the eager, single-threaded result bit for bit."""
import threading

import numpy as np
import pytest
import torch

import svod_amd
from svod_amd import Attn, KeyMask, Qkv
from util import Lcg, bf16_tensor, bits

pytestmark = pytest.mark.gpu


def layer(qkv, tables, w, lens, order, residual, norm_w, outs=None):
    """A model layer's calls on this path: prologue, ordered attention, a split decoder-style call, a norm."""
    h, hkv, d = 8, 4, 64
    q, k, v = svod_amd.heads(qkv, Qkv(h, hkv, d, w, w, 1e-6, tables), out=None if outs is None else outs["qkv"])
    svod_amd.order_rows(lens, out=order)
    o = svod_amd.attention(q, k, v, Attn(causal=True, keys=KeyMask.lens(lens), row_order=order),
                           out=None if outs is None else outs["o"])
    step = svod_amd.attention(q[:, :1].contiguous() if outs is None else outs["q1"].copy_(q[:, :1]), k, v,
                              Attn(keys=KeyMask.lens(lens), splits=3),
                              out=None if outs is None else outs["step"], workspace=None if outs is None else outs["ws"])
    s, y = svod_amd.add_rms_norm(o.view(o.shape[0], o.shape[1], h * d), residual, norm_w, 1e-5,
                                 out=None if outs is None else outs["norm"])
    return q, k, v, o, step, s, y


def inputs(device, seed):
    g = Lcg(seed)
    b, t, h, hkv, d = 4, 300, 8, 4, 64
    qkv = bf16_tensor(g.bf16((b, t, (h + 2 * hkv) * d), mul=3.0), device)
    cos, sin = (bf16_tensor(g.bf16((1, t, 1, d // 2)), device) for _ in range(2))
    w = bf16_tensor(g.bf16((d,), mul=0.5, add=1.0), device)
    residual = bf16_tensor(g.bf16((b, t, h * d)), device)
    norm_w = bf16_tensor(g.bf16((h * d,), mul=0.5, add=1.0), device)
    lens = torch.tensor([t, 70 + seed, 1, 255], dtype=torch.int32, device=device)
    return qkv, (cos, sin), w, lens, residual, norm_w


def test_a_captured_layer_replays_to_the_eager_result(device):
    first = inputs(device, 5)
    qkv, tables, w, lens, residual, norm_w = (x.clone() if torch.is_tensor(x) else tuple(y.clone() for y in x) for x in first)
    order = torch.empty(4, dtype=torch.int32, device=device)
    eager = layer(qkv, tables, w, lens, order, residual, norm_w)  # also the first use of these kernels
    torch.cuda.synchronize()
    outs = {"qkv": tuple(torch.empty_like(x) for x in eager[:3]), "o": torch.empty_like(eager[3]),
            "q1": torch.empty_like(eager[0][:, :1].contiguous()), "step": torch.empty_like(eager[4]),
            # the partial states of three splits: (o [D], m, l) in f32 per split, batch row, query and head
            "ws": torch.empty(3 * 4 * 1 * 8 * (64 + 2) * 4, dtype=torch.uint8, device=device),
            "norm": (torch.empty_like(eager[5]), torch.empty_like(eager[6]))}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        layer(qkv, tables, w, lens, order, residual, norm_w, outs)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = layer(qkv, tables, w, lens, order, residual, norm_w, outs)
    for seed in (5, 6, 7, 5):
        fresh = inputs(device, seed)
        qkv.copy_(fresh[0]); tables[0].copy_(fresh[1][0]); tables[1].copy_(fresh[1][1]); w.copy_(fresh[2])
        lens.copy_(fresh[3]); residual.copy_(fresh[4]); norm_w.copy_(fresh[5])
        for x in captured:
            x.fill_(3.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = layer(*fresh[:4], torch.empty_like(order), *fresh[4:])
        torch.cuda.synchronize()
        for got, ref, name in zip(captured, want, ("q", "k", "v", "o", "step", "sum", "norm")):
            assert np.array_equal(bits(got), bits(ref)), (seed, name)


def test_threads_launch_side_by_side(device):
    """Four host threads, a stream each, different shapes and options: the same bits as one thread, and
    each thread's `chosen()` is its own (tk/src/ops/mod.rs:83-118: thread-local)."""
    cases = [(2, 200, 200, 4, 4, 64, True, None), (1, 130, 260, 8, 2, 128, False, None),
             (3, 64, 500, 4, 2, 64, False, 4), (2, 96, 96, 2, 2, 32, True, None)]

    def operands(i):
        b, t, tk, h, hkv, d, causal, splits = cases[i]
        g = Lcg(10 + i)
        q, k, v = (bf16_tensor(g.bf16(s), device) for s in ((b, t, h, d), (b, tk, hkv, d), (b, tk, hkv, d)))
        lens = torch.tensor([tk - 7 * j for j in range(b)], dtype=torch.int32, device=device)
        return q, k, v, Attn(causal=causal, keys=KeyMask.lens(lens), splits=splits)

    want, names = [], []
    for i in range(4):
        q, k, v, opts = operands(i)
        want.append(bits(svod_amd.attention(q, k, v, opts)))
        names.append(svod_amd.chosen())
    torch.cuda.synchronize()
    errors = []

    def work(i):
        try:
            torch.cuda.set_device(device)
            q, k, v, opts = operands(i)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for _ in range(40):
                    got = svod_amd.attention(q, k, v, opts)
                    assert svod_amd.chosen() == names[i], (svod_amd.chosen(), names[i])
                stream.synchronize()
            assert np.array_equal(bits(got), want[i]), i
        except Exception as e:  # noqa: BLE001 - reported by the parent
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(timeout=100)
    assert not errors, errors
    assert not any(th.is_alive() for th in threads)
