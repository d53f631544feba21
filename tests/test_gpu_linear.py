"""The GEMM with the rope epilogue through the C ABI (tk/src/ops/linear.rs:60-231, tk/src/kernels/gemm.rs:604-716),
against the oracle: the reference's own cases (tk/src/test/unit/ops.rs:291-340: turned_linear_matches_the_graph,
turned_linear_under_a_batch_variable) held to the reference's bar (rel 2e-2 against the unrounded f64 epilogue),
then Qwen3's projection shape on sampled rows, and the path the epilogue exists for: the turned projection read in
place by attention_packed equals the prologue's output fed to attention."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, Fallback, GraphFallback, Linear, Qkv, Rotary
from util import Lcg, assert_rel_close, bf16_tensor, bits, max_abs, mean_rel, to_np

pytestmark = pytest.mark.gpu


def tables(t, d, device, theta=10_000.0):
    cos, sin = oracle.rope_table(theta, t, d)
    cos, sin = oracle.round_bf16(cos), oracle.round_bf16(sin)
    dev = lambda a: bf16_tensor(a.reshape(1, t, 1, d // 2), device)
    return (cos, sin), (dev(cos), dev(sin))


def case(lead, k, n, seed=40):
    g = Lcg(seed)
    return g.bf16((*lead, k)), g.bf16((n, k), mul=0.3), g.bf16((n,))


# (name, lead, [h, h_kv, d], bias, k): ops.rs:296-298
TURNED = [
    ("grouped heads, partial rows", (2, 37), (4, 2, 64), False, 128),
    ("ModernBERT's heads under a bias", (1, 100), (12, 12, 64), True, 128),
    ("d 128", (3, 16), (2, 1, 128), False, 128),
    ("an odd count of turned heads of 64", (2, 50), (2, 1, 64), True, 96),
    ("rows and columns across tiles", (2, 300), (4, 2, 128), True, 256),
    ("a k loop of one stage", (2, 40), (2, 2, 64), True, 32),
    ("a k loop of two stages, shorter than the ring", (1, 300), (2, 1, 128), False, 64),
]


@pytest.mark.parametrize("name,lead,heads,bias,k", TURNED, ids=[c[0] for c in TURNED])
def test_turned_linear_matches_the_reference(device, name, lead, heads, bias, k):
    h, hkv, d = heads
    n = (h + 2 * hkv) * d
    x, w, bv = case(lead, k, n)
    (cos, sin), (cos_d, sin_d) = tables(lead[1], d, device)
    y = svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device),
                        Linear(bias=bf16_tensor(bv, device) if bias else None, rope=Rotary(cos_d, sin_d, h + hkv, d)))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "linear", family: "gemm"') and "rope" in svod_amd.chosen()
    want = oracle.linear_direct(x, w, bv if bias else None, (cos, sin, h + hkv, d))
    assert_rel_close(name, to_np(y), want, 2e-2)  # ops.rs:312
    # One rounding at the store: against the f64 result as bf16 stores it nearly every element is the same bits.
    assert mean_rel(to_np(y), oracle.round_bf16(want.astype(np.float32))) < 2e-4
    # and against the kernel's arithmetic restated in f32, closer still
    assert mean_rel(to_np(y), oracle.linear_kernel(x, w, bv if bias else None, (cos, sin, h + hkv, d))) < 2e-4


def test_plain_linear_and_f16(device):
    x, w, bv = case((3, 50), 64, 96, seed=7)
    y = svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device), Linear(bias=bf16_tensor(bv, device)))
    torch.cuda.synchronize()
    assert_rel_close("plain", to_np(y), oracle.linear_direct(x, w, bv), 2e-2)
    xh, wh = (torch.from_numpy(oracle.round_f16(a)).to(torch.float16).to(device) for a in (x, w))
    (cos, sin), _ = tables(50, 32, device)
    y16 = svod_amd.linear(xh, wh)
    torch.cuda.synchronize()
    f = lambda t: t.detach().cpu().to(torch.float32).numpy()
    assert_rel_close("f16", f(y16), oracle.linear_direct(f(xh), f(wh)), 2e-2)


def test_turned_linear_under_a_bound_batch(device):
    """ops.rs:319-340: live batches below the capacity; rows past them are not written."""
    cap, live, t, (h, hkv, d), k = 4, 3, 37, (4, 2, 64), 128
    n = (h + 2 * hkv) * d
    x, w, _ = case((cap, t), k, n, seed=43)
    (cos, sin), (cos_d, sin_d) = tables(t, d, device)
    out = torch.full((cap, t, n), float("nan"), dtype=torch.bfloat16, device=device)
    svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device),
                    Linear(rope=Rotary(cos_d, sin_d, h + hkv, d), batch_live=live), out=out)
    torch.cuda.synchronize()
    want = oracle.linear_direct(x[:live], w, None, (cos, sin, h + hkv, d))
    assert_rel_close("bound batch", to_np(out[:live]), want, 2e-2)
    assert torch.isnan(out[live:]).all()


def test_what_the_kernel_does_not_hold_keeps_the_graph(device):
    x, w, bv = case((2, 37), 128, 512)
    xd, wd = bf16_tensor(x, device), bf16_tensor(w, device)
    (_, _), (cos_d, sin_d) = tables(37, 32, device)
    for opts, why in ((Linear(act=svod_amd.Act.Gelu), Fallback.Config), (Linear(scale=0.5), Fallback.Config),
                      (Linear(rope=Rotary(cos_d, sin_d, 4, 32)), Fallback.Config)):  # heads of 32: no tile turns them
        with pytest.raises(GraphFallback) as e:
            svod_amd.linear(xd, wd, opts)
        assert e.value.why == why
    (_, _), (c64, s64) = tables(37, 64, device)
    with pytest.raises(GraphFallback) as e:  # tables off the stream dtype (ops.rs:299)
        svod_amd.linear(xd, wd, Linear(rope=Rotary(c64.float(), s64.float(), 4, 64)))
    assert e.value.why == Fallback.Dtype
    with pytest.raises(GraphFallback) as e:  # k-columns not in whole stages
        svod_amd.linear(bf16_tensor(x[:, :, :100], device), bf16_tensor(w[:, :100], device))
    assert e.value.why == Fallback.Shape


def test_qwen3_projection_shape_on_sampled_rows(device):
    """The projection of the Qwen3-shaped workload, [8*2048, 1024] x [4096, 1024], heads of 128 turned: sampled
    rows against the oracle, and linearity as the size-independent property (y(x1 + x2) = y(x1) + y(x2) to rounding)."""
    b, t, k, h, hkv, d = 8, 2048, 1024, 16, 8, 128
    n = (h + 2 * hkv) * d
    g = torch.Generator(device=device).manual_seed(5)
    x = torch.randn((b, t, k), generator=g, device=device).to(torch.bfloat16)
    w = (torch.randn((n, k), generator=g, device=device) * (1.0 / 32)).to(torch.bfloat16)
    (cos, sin), (cos_d, sin_d) = tables(t, d, device, theta=1e6)
    y = svod_amd.linear(x, w, Linear(rope=Rotary(cos_d, sin_d, h + hkv, d)))
    torch.cuda.synchronize()
    rows = [(0, 0), (0, 1), (3, 1027), (7, 2047), (5, 255), (5, 256)]
    wn = to_np(w)
    for bi, ti in rows:
        want = oracle.linear_direct(to_np(x[bi:bi + 1, ti:ti + 1]), wn, None, (cos[ti:ti + 1], sin[ti:ti + 1], h + hkv, d))
        assert_rel_close(f"row {bi},{ti}", to_np(y[bi, ti]), want[0, 0], 2e-2)
    half = (x.float() * 0.5).to(torch.bfloat16)  # exact
    y_half = svod_amd.linear(half, w, Linear(rope=Rotary(cos_d, sin_d, h + hkv, d)))
    torch.cuda.synchronize()
    assert float((y_half.float() * 2 - y.float()).abs().max()) <= float(y.float().abs().max()) * 2 ** -7


def test_the_turned_projection_feeds_attention_in_place(device):
    """What the epilogue is for (tk/src/ops/linear.rs:47-58, tk/src/ops/attention.rs:104-122): linear with the rope,
    then attention_packed on its output, against projection -> prologue (rope only) -> attention."""
    b, t, k, h, hkv, d = 2, 200, 256, 4, 2, 64
    n = (h + 2 * hkv) * d
    x, w, _ = case((b, t), k, n, seed=9)
    (cos, sin), (cos_d, sin_d) = tables(t, d, device)
    xd, wd = bf16_tensor(x, device), bf16_tensor(w * 0.3, device)
    fused = svod_amd.linear(xd, wd, Linear(rope=Rotary(cos_d, sin_d, h + hkv, d)))
    a = svod_amd.attention_packed(fused, h, hkv, Attn(causal=True))
    plain = svod_amd.linear(xd, wd)
    q, kk, v = svod_amd.heads(plain, Qkv(h, hkv, d, None, None, 1e-6, (cos_d, sin_d)))
    bref = svod_amd.attention(q, kk, v, Attn(causal=True))
    torch.cuda.synchronize()
    # The two differ by one more rounding of q and k (the prologue rotates rounded values): within the op's bar.
    assert max_abs(to_np(a), to_np(bref)) < 2e-2
    assert np.array_equal(bits(fused[:, :, (h + hkv) * d:]), bits(plain[:, :, (h + hkv) * d:]))  # values: as they are


def test_into_stores_a_window_of_a_wider_output(device):
    """Linear::into (tk/src/ops/linear.rs:40-42, tk/src/ops/mod.rs:459-477): the result lands in channels
    at .. at + N of the caller's [lead..., C] tensor, bit-equal to the plain call's, the rest untouched; a window
    the 16-byte stores cannot land in keeps the graph; one that does not fit is a shape error."""
    lead, k, n, c, at = (2, 70), 96, 3 * 64, 512, 128
    x, w, bv = case(lead, k, n)
    (cos, sin), (cos_d, sin_d) = tables(lead[1], 64, device)
    opts = dict(bias=bf16_tensor(bv, device), rope=Rotary(cos_d, sin_d, 2, 64))
    want = svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device), Linear(**opts))
    wide = torch.full((*lead, c), 3.0, dtype=torch.bfloat16, device=device)
    got = svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device), Linear(into=(wide, at), **opts))
    torch.cuda.synchronize()
    assert got is wide and svod_amd.chosen().startswith('Kernel { op: "linear"')
    assert np.array_equal(bits(wide[..., at:at + n].contiguous()), bits(want))
    assert bool((wide[..., :at] == 3.0).all()) and bool((wide[..., at + n:] == 3.0).all())
    with pytest.raises(GraphFallback) as e:
        svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device), Linear(into=(wide, 4), **opts))
    assert e.value.why == Fallback.Config
    with pytest.raises(svod_amd.OpError) as e:
        svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device), Linear(into=(wide, c - n + 8), **opts))
    assert e.value.kind == "Shape"


@pytest.fixture
def tile_by_shape():
    yield
    svod_amd.tune_linear(0)


@pytest.mark.parametrize("lead,heads,k,bias", [((2, 300), (4, 2, 128), 256, True), ((1, 37), (12, 12, 64), 96, False),
                                               ((3, 129), None, 160, True), ((1, 1), None, 32, False)],
                         ids=["turned 128 across tiles", "turned 64, partial rows", "plain across tiles", "one row"])
def test_the_two_tiles_give_the_same_bits(device, tile_by_shape, lead, heads, k, bias):
    """svodk_tune_linear: 128 x 128 tiles by 4 waves against 256 x 256 by 8; a column's k-steps are summed in the
    same order, so nothing but the launch differs."""
    n = (heads[0] + 2 * heads[1]) * heads[2] if heads else 8 * 41
    x, w, bv = case(lead, k, n, seed=51)
    opts = dict(bias=bf16_tensor(bv, device)) if bias else {}
    if heads:
        _, (cos_d, sin_d) = tables(lead[1], heads[2], device)
        opts["rope"] = Rotary(cos_d, sin_d, heads[0] + heads[1], heads[2])
    got = {}
    for tile in (256, 128):
        svod_amd.tune_linear(tile)
        got[tile] = svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device), Linear(**opts))
        torch.cuda.synchronize()
        assert f"bm: {tile}, bn: {tile}" in svod_amd.chosen(), svod_amd.chosen()
    assert np.array_equal(bits(got[256]), bits(got[128]))


def test_the_tile_follows_the_shape(device, tile_by_shape):
    """Few rows take 128 x 128 tiles (four times the workgroups), a product that fills the part 256 x 256."""
    svod_amd.tune_linear(0)
    w = bf16_tensor(np.ones((4096, 64), dtype=np.float32), device)
    for rows, tile in ((512, 128), (2048, 128), (4096, 256), (16384, 256)):
        svod_amd.linear(bf16_tensor(np.ones((rows, 64), dtype=np.float32), device), w)
        torch.cuda.synchronize()
        assert f"bm: {tile}, bn: {tile}" in svod_amd.chosen(), (rows, svod_amd.chosen())
