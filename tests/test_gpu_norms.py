"""Row norms (tk/src/ops/norm.rs:16-42, tk/src/kernels/rows.rs:41-115) through the C ABI against the oracle.
The cases are the reference's own: the device tests of tk/src/test/unit/rows.rs:232-256 (37 rows: a partial
last block; out within 1e-2 relative of the f64 reference, the fused sum exact) and the op tests of
tk/src/test/unit/ops.rs:702-749 (against the graph within 2e-2, a bound batch), then wider rows."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from util import Lcg, bf16_tensor, bits, to_np

pytestmark = pytest.mark.gpu

LAYER, RMS = oracle.LAYER, oracle.RMS


def inputs(rows_shape, d, seed=5):
    """norm_inputs of tk/src/test/unit/rows.rs:147-165."""
    g = Lcg(seed)
    shape = tuple(rows_shape) + (d,)
    return g.bf16(shape, mul=2.0, add=1.5), g.bf16(shape), g.bf16((d,), mul=0.5, add=1.0), g.bf16((d,), mul=0.5)


def run(device, kind, rows_shape, d, residual, bias, eps, f16=False, batch_live=None):
    x, r, w, b = inputs(rows_shape, d)
    if f16:
        x, r, w, b = (oracle.round_f16(a) for a in (x, r, w, b))
        up = lambda a: torch.from_numpy(a).to(torch.float16).to(device)
    else:
        up = lambda a: bf16_tensor(a, device)
    bb = up(b) if (bias and kind == LAYER) else None
    if kind == LAYER:
        got = (svod_amd.add_layer_norm(up(x), up(r), up(w), bb, eps, batch_live=batch_live) if residual
               else svod_amd.layer_norm(up(x), up(w), bb, eps, batch_live=batch_live))
    else:
        got = (svod_amd.add_rms_norm(up(x), up(r), up(w), eps, batch_live=batch_live) if residual
               else svod_amd.rms_norm(up(x), up(w), eps, batch_live=batch_live))
    torch.cuda.synchronize()
    name = "layer_norm" if kind == LAYER else "rms_norm"
    assert svod_amd.chosen() == 'Kernel { op: "%s", family: "%s", cfg: "NormCfg { br: 4 }" }' % (name, name), svod_amd.chosen()
    want = oracle.norm_direct(kind, x, w, b if (bias and kind == LAYER) else None, residual=r if residual else None, eps=eps)
    return got, want, (x, r, w, b)


def close(got, want, tol):
    return np.all(np.abs(got.astype(np.float64) - want) <= tol * np.maximum(np.abs(want), 1.0))


# rows.rs:232-239 and ops.rs:702-708
CASES = [
    ("layer 512", LAYER, 512, False, True), ("layer 512 without a bias", LAYER, 512, False, False),
    ("layer 1024 residual", LAYER, 1024, True, True), ("rms 512 residual", RMS, 512, True, False),
    ("rms 1024", RMS, 1024, False, False), ("rms 2048", RMS, 2048, False, False),
    ("layer 768 without a bias, a span and a half", LAYER, 768, False, False), ("add layer 256", LAYER, 256, True, True),
    ("layer 1024", LAYER, 1024, False, True), ("add rms 1024", RMS, 1024, True, False),
    ("rms 4096, past the reference's widest", RMS, 4096, True, False), ("layer 3840", LAYER, 3840, True, True),
    ("rms 1280", RMS, 1280, False, False),
]


@pytest.mark.parametrize("name,kind,d,residual,bias", CASES, ids=[c[0] for c in CASES])
def test_norms_match_the_f64_reference(device, name, kind, d, residual, bias):
    eps = 1e-5 if kind == LAYER else 1e-6
    got, (want, want_sum), _ = run(device, kind, (37,), d, residual, bias, eps)
    out = to_np(got[1] if residual else got)
    assert close(out, oracle.round_bf16(want), 1e-2)  # rows.rs:250-251
    if residual:
        assert np.array_equal(to_np(got[0]), want_sum)  # rows.rs:252-254: the sum is exact


@pytest.mark.parametrize("kind,residual", [(LAYER, True), (RMS, False)])
def test_norms_match_the_graph(device, kind, residual):
    """ops.rs:722-729: within 2e-2 of the graph's f32 arithmetic."""
    got, _, (x, r, w, b) = run(device, kind, (3, 37), 1024, residual, True, 1e-5)
    graph, graph_sum = oracle.norm_f32(kind, x, w, b if kind == LAYER else None, residual=r if residual else None, eps=1e-5)
    assert close(to_np(got[1] if residual else got), graph, 2e-2)
    if residual:
        assert np.array_equal(to_np(got[0]), graph_sum)


def test_f16_rms_256(device):
    """ops.rs:708."""
    got, (want, _), _ = run(device, RMS, (37,), 256, False, False, 1e-6, f16=True)
    assert close(got.detach().cpu().to(torch.float32).numpy(), want, 1e-2)


def test_norm_under_a_batch_variable(device):
    """ops.rs:731-749: of four batches of capacity three are live; the fourth is not written."""
    cap, live, d = 4, 3, 512
    x, r, w, b = inputs((cap, 37), d, seed=40)
    dx, dr, dw, db = (bf16_tensor(a, device) for a in (x, r, w, b))
    total = torch.full_like(dx, 7.0)
    y = torch.full_like(dx, 7.0)
    svod_amd.add_layer_norm(dx, dr, dw, db, 1e-5, out=(total, y), batch_live=live)
    torch.cuda.synchronize()
    want, want_sum = oracle.norm_direct(LAYER, x[:live], w, b, residual=r[:live], eps=1e-5)
    assert close(to_np(y)[:live], oracle.round_bf16(want), 1e-2)
    assert np.array_equal(to_np(total)[:live], want_sum)
    assert (to_np(y)[live:] == 7.0).all() and (to_np(total)[live:] == 7.0).all()


def test_closed_forms(device):
    d = 1024
    ones = bf16_tensor(np.ones(d, dtype=np.float32), device)
    row = bf16_tensor(np.full((5, d), 3.0, dtype=np.float32), device)
    got = to_np(svod_amd.rms_norm(row, ones, 1e-6))
    assert np.array_equal(got, np.ones_like(got))  # 3 / sqrt(9 + 1e-6) rounds to 1
    quarter = bf16_tensor(np.full(d, 0.25, dtype=np.float32), device)
    got = to_np(svod_amd.layer_norm(row, ones, quarter, 1e-5))
    assert np.array_equal(got, np.full_like(got, 0.25))  # a constant row centres to zero: the bias is left
    x = bf16_tensor(inputs((9,), d)[0], device)
    y = to_np(svod_amd.layer_norm(x, ones, None, 1e-5)).astype(np.float64)
    assert np.abs(y.mean(-1)).max() < 5e-3 and np.abs(y.var(-1) - 1.0).max() < 2e-2


def test_many_rows_and_the_same_bits_whatever_the_row_count(device):
    """A row's arithmetic does not depend on its neighbours: the first rows of a long input come out
    as they do alone."""
    d = 2048
    x, r, w, _ = inputs((1000,), d, seed=11)
    dw = bf16_tensor(w, device)
    many = svod_amd.add_rms_norm(bf16_tensor(x, device), bf16_tensor(r, device), dw, 1e-6)
    few = svod_amd.add_rms_norm(bf16_tensor(x[:5], device), bf16_tensor(r[:5], device), dw, 1e-6)
    assert np.array_equal(bits(many[1])[:5], bits(few[1]))
    assert np.array_equal(bits(many[0])[:5], bits(few[0]))
    want, _ = oracle.norm_direct(RMS, x, w, residual=r, eps=1e-6)
    assert close(to_np(many[1]), oracle.round_bf16(want), 1e-2)


def test_the_stored_sum_rounds_as_the_reference_does_at_the_edges(device):
    """tk/src/interp.rs:37-44 where a plausible narrowing differs: ties to even in both directions, the carry
    into the exponent, the largest finite value's overflow to infinity, subnormals, signed zeros, infinities and
    the bits of a NaN; every pair of bf16 values of a sweep as well (x + r in f32, narrowed once)."""
    d = 256
    x16 = np.array([0x3F80, 0x3F81, 0x3F80, 0x3FFF, 0x7F7F, 0x7F7F, 0xFF7F, 0x0001, 0x0001, 0x8001, 0x0000, 0x8000,
                    0x7F80, 0x7F80, 0x7FC1, 0xFFA0, 0x0080, 0x4000], dtype=np.uint16)
    r16 = np.array([0x3B80, 0x3B80, 0x3B00, 0x3B80, 0x7300, 0x7B00, 0xFB00, 0x0001, 0x8001, 0x8002, 0x8000, 0x8000,
                    0xFF80, 0x3F80, 0x3F80, 0x0000, 0x8001, 0x3780], dtype=np.uint16)
    g = np.random.default_rng(21)
    sweep = g.integers(0, 1 << 16, size=(2, 64 * d - x16.size), dtype=np.uint16)
    x = oracle.from_bf16_bits(np.concatenate([x16, sweep[0]])).reshape(64, d)
    r = oracle.from_bf16_bits(np.concatenate([r16, sweep[1]])).reshape(64, d)
    up = lambda a: torch.from_numpy((a.view(np.uint32) >> 16).astype(np.uint16).view(np.int16)).view(torch.bfloat16).to(device)
    total, _ = svod_amd.add_rms_norm(up(x), up(r), bf16_tensor(np.ones(d, dtype=np.float32), device), 1e-6)
    torch.cuda.synchronize()
    with np.errstate(all="ignore"):
        want = oracle.bf16_bits(x + r)
        nan = np.isnan(x + r)
    got = bits(total)
    assert np.array_equal(got[~nan], want[~nan])
    # A NaN keeps being one, quiet; which operand's payload the f32 add carries over is the adder's business.
    assert ((got[nan] & 0x7FC0) == 0x7FC0).all()
    assert nan.sum() > 100 and (~nan).sum() > 10000


def test_a_form_first_met_under_stream_capture(device):
    """The launch asks the runtime once per form what a compute unit holds; that question is allowed while a
    stream is being captured, and the captured launch gives the eager call's bits on every replay."""
    d = 3328  # a width and form no other test of this process runs: f16, LayerNorm, residual, bias
    g = np.random.default_rng(3)
    mk = lambda *shape: torch.from_numpy(g.standard_normal(shape).astype(np.float32)).to(torch.float16).to(device)
    x, r, w, b = mk(301, d), mk(301, d), mk(d), mk(d)
    total, y = torch.empty_like(x), torch.empty_like(x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            svod_amd.add_layer_norm(x, r, w, b, 1e-5, out=(total, y))
    torch.cuda.current_stream().wait_stream(side)
    seen = []
    for _ in range(3):
        total.zero_(), y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        seen.append((total.clone(), y.clone()))
    eager = svod_amd.add_layer_norm(x, r, w, b, 1e-5)
    torch.cuda.synchronize()
    for t, o in seen:
        assert torch.equal(t, eager[0]) and torch.equal(o, eager[1])


def test_a_width_without_a_kernel_keeps_the_graph(device):
    x = bf16_tensor(np.ones((4, 1000), dtype=np.float32), device)
    with pytest.raises(svod_amd.GraphFallback) as e:
        svod_amd.rms_norm(x, bf16_tensor(np.ones(1000, dtype=np.float32), device))
    assert e.value.why == svod_amd.Fallback.Shape
    assert svod_amd.chosen() == 'Graph { op: "rms_norm", why: Shape }'
