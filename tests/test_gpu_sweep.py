"""A seeded sweep over the options of one attention call taken together (tk/src/ops/attention.rs:60-86): head
sizes, GQA groups, query and key counts around the tile and block edges, causal, windows, chunk masks, segment
starts, key lengths and key masks, an additive bias, key splits, scales, both 16-bit types.  The named cases of the
other modules take the options one or two at a time; here every call draws all of them, and every result is held
against the float64 direct softmax of the same operands (tk/src/test/unit/attention.rs:102-178) to the op's bar."""
import random

import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import assert_bf16_parity, assert_rel_close, max_abs, to_np

# The tile program is what the sweep holds the results against: the decoder step's own kernel has a sweep of its own.
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("key_tiles")]


def draw(rng: random.Random, f16: bool, shape, sigma=1.0):
    """Values exact in the call's 16-bit type, as float32."""
    x = np.asarray([rng.gauss(0.0, sigma) for _ in range(int(np.prod(shape)))], dtype=np.float32).reshape(shape)
    return oracle.round_f16(x) if f16 else oracle.round_bf16(x)


def one_call(rng: random.Random, device):
    d = rng.choice([32, 48, 64, 64, 128, 128, 256])
    hkv = rng.choice([1, 2, 3])
    h = hkv * rng.choice([1, 1, 2, 4])
    b = rng.choice([1, 2, 3])
    t = rng.choice([1, 7, 31, 64, 65, 127, 128, 129, 200, 257, 333])
    tk = t if rng.random() < 0.6 else rng.choice([1, 5, 63, 64, 65, 128, 191, 300, 400])
    f16 = rng.random() < 0.25
    opts, prob = {}, {}
    if rng.random() < 0.4:
        opts["causal"] = prob["causal"] = True
    ranged = rng.random()
    if ranged < 0.2:
        opts["window"] = prob["window"] = (rng.choice([0, 3, 40, 150]), rng.choice([0, 0, 5, 70]))
    elif ranged < 0.4:
        opts["chunk"] = prob["chunk"] = (rng.choice([1, 8, 24, 64, 100]), rng.choice([None, 0, 1, 3]), rng.choice([0, 0, 1, 2]))
    if t == tk and rng.random() < 0.25:
        length = rng.choice([1, 17, 40, 64, 130])
        seg = np.tile(np.arange(t) - np.arange(t) % length, (b, 1))
        opts["seg_start"] = torch.from_numpy(seg).to(rng.choice([torch.int32, torch.int64])).to(device)
        prob["seg_start"] = seg
    keys = rng.choice(["none", "lens", "mask"])
    if keys == "lens":
        lens = np.asarray([rng.choice([0, 1, tk, tk // 2, max(tk - 1, 0), rng.randint(0, tk)]) for _ in range(b)])
        opts["keys"] = KeyMask.lens(torch.from_numpy(lens).to(rng.choice([torch.int32, torch.int64])).to(device))
        prob["key_lens"] = lens
    elif keys == "mask":
        mask = np.asarray([[rng.random() < 0.7 for _ in range(tk)] for _ in range(b)])
        if b > 1:
            mask[1] = False
        opts["keys"] = KeyMask.bool(torch.from_numpy(mask).to(device))
        prob["key_mask"] = mask
    scale = rng.choice([None, None, 0.05, 0.3])
    if scale is not None:
        opts["scale"] = prob["scale"] = scale
    q, k, v = draw(rng, f16, (b, t, h, d)), draw(rng, f16, (b, tk, hkv, d)), draw(rng, f16, (b, tk, hkv, d))
    dt = torch.float16 if f16 else torch.bfloat16
    up = lambda a: torch.from_numpy(a).to(dt).to(device)
    if rng.random() < 0.2:
        bias = draw(rng, f16, (rng.choice([1, b]), h, t, tk), sigma=2.0)
        opts["bias"], prob["bias"] = up(bias), bias
    splits = rng.choice([None, None, None, 2, 3])
    name = (f"b{b} t{t} tk{tk} h{h}/{hkv} d{d} {'f16' if f16 else 'bf16'} splits={splits} keys={keys} "
            + " ".join(f"{key}={val if not hasattr(val, 'shape') else 'yes'}" for key, val in prob.items() if key not in ("key_lens", "key_mask")))
    # Splits are the caller's here (without a lent workspace the library names none of its own), so the
    # reference's program can be run with the same count.
    workspace = None if splits is None else torch.empty(splits * b * t * h * (d + 2) * 4, dtype=torch.uint8, device=device)
    try:
        got = svod_amd.attention(up(q), up(k), up(v), Attn(splits=splits, **opts), workspace=workspace)
    except svod_amd.GraphFallback as e:
        return name, None, str(e), None, f16
    torch.cuda.synchronize()
    problem = oracle.AttnProblem(q, k, v, bf16=not f16, **prob)
    direct = oracle.attention_direct(problem, threads=8)
    count = min(splits or 1, max(1, (tk + 63) // 64))
    if f16:
        with oracle.stream_dtype("f16"):
            program = oracle.attention_flash(problem, bq=128, bkv=64, splits=count)
    else:
        program = oracle.attention_flash(problem, bq=128, bkv=64, splits=count)
    return name, got, direct, program, f16


def test_calls_that_draw_every_option_match_the_direct_softmax(device):
    rng = random.Random(41)
    ran, kept_graph = 0, []
    for case in range(150):
        name, got, direct, program, f16 = one_call(rng, device)
        name = f"case {case}: {name}"
        if got is None:
            kept_graph.append((name, direct))
            continue
        ran += 1
        g = to_np(got)
        if f16:
            assert np.isfinite(g).all(), name
            assert max_abs(g, direct) < 2e-2, name   # attention.rs:483
            assert_rel_close(name, g, program, 2e-3)  # the program's f32 result; an f16 store is within 2^-11 of it
        else:
            assert_bf16_parity(name, g, direct, program)
    # A call keeps the graph only for what the library states it has no kernel for.
    for name, why in kept_graph:
        assert "Config" in why or "Shape" in why, (name, why)
    assert ran >= 130, (ran, kept_graph[:5])


def test_projections_that_draw_every_option_match_the_reference(device):
    """The GEMM with its epilogue over row, column and k counts on and off the 256 x 256 tile, the two-step last
    stage, biases, turned heads of 64 and 128 and windows of a wider output (tk/src/ops/linear.rs:24-58), held to
    the reference's bar against the unrounded f64 epilogue (tk/src/test/unit/ops.rs:312)."""
    from svod_amd import Linear, Rotary
    from util import Lcg, assert_rel_close, bf16_tensor, bits, mean_rel
    rng = random.Random(43)
    for case in range(60):
        d = rng.choice([64, 128])
        hq, hk = rng.choice([1, 2, 4, 6]), rng.choice([1, 2])
        turned = rng.random() < 0.6
        n = (hq + 2 * hk) * d if turned else 8 * rng.choice([1, 5, 32, 33, 63, 100])
        batch, t = rng.choice([1, 2, 3]), rng.choice([1, 9, 37, 128, 255, 257, 300])
        k = 32 * rng.choice([1, 2, 3, 4, 5, 8, 13])
        g = Lcg(100 + case)
        x, w, bv = g.bf16((batch, t, k)), g.bf16((n, k), mul=0.3), g.bf16((n,))
        bias = rng.random() < 0.5
        opts, rope = {}, None
        if bias:
            opts["bias"] = bf16_tensor(bv, device)
        if turned:
            cos, sin = oracle.rope_table(10_000.0, t, d)
            cos, sin = oracle.round_bf16(cos), oracle.round_bf16(sin)
            heads = rng.choice([hq + hk, hq, 1])
            opts["rope"] = Rotary(bf16_tensor(cos.reshape(1, t, 1, d // 2), device), bf16_tensor(sin.reshape(1, t, 1, d // 2), device), heads, d)
            rope = (cos, sin, heads, d)
        name = f"case {case}: rows {batch}x{t} n {n} k {k} bias={bias} rope={None if rope is None else rope[2:]}"
        wide = None
        if rng.random() < 0.3:
            at = 8 * rng.choice([0, 1, 16])
            wide = torch.full((batch, t, n + at + 8 * rng.choice([0, 3])), 3.0, dtype=torch.bfloat16, device=device)
            opts["into"] = (wide, at)
        svod_amd.tune_linear((256, 128, 0)[case % 3])  # both tiles, and the shape's own choice
        try:
            y = svod_amd.linear(bf16_tensor(x, device), bf16_tensor(w, device), Linear(**opts))
            torch.cuda.synchronize()
        finally:
            svod_amd.tune_linear(0)
        assert svod_amd.chosen().startswith('Kernel { op: "linear", family: "gemm"'), (name, svod_amd.chosen())
        if wide is not None:
            assert y is wide, name
            assert bool((wide[..., :at] == 3.0).all()) and bool((wide[..., at + n:] == 3.0).all()), name
            y = wide[..., at:at + n].contiguous()
        want = oracle.linear_direct(x, w, bv if bias else None, rope)
        assert_rel_close(name, to_np(y), want, 2e-2)
        assert mean_rel(to_np(y), oracle.round_bf16(want.astype(np.float32))) < 3e-4, name


def test_prologues_that_draw_every_option_match_the_reference(device):
    """The prologue over head counts, head sizes, row counts, either norm, rotary tables by position or by token,
    both 16-bit types' worth of values (tk/src/ops/heads.rs:19-31) to the bars of tk/src/test/unit/heads.rs:124,159."""
    from svod_amd import Qkv
    from util import Lcg, bf16_tensor, bits
    rng = random.Random(44)
    for case in range(60):
        d = rng.choice([16, 32, 64, 64, 128, 128, 256])
        hk = rng.choice([1, 2, 3, 8])
        hq = hk * rng.choice([1, 2, 4])
        batch, t = rng.choice([1, 2, 3]), rng.choice([1, 5, 37, 64, 130, 257])
        norms = (rng.random() < 0.6, rng.random() < 0.6)
        rope = rng.choice([None, False, True])
        g = Lcg(200 + case)
        slots, half = hq + 2 * hk, d // 2
        qkv = g.bf16((batch, t, slots * d), mul=3.0)
        q_w = g.bf16((d,), mul=0.5, add=1.0) if norms[0] else None
        k_w = g.bf16((d,), mul=0.5, add=1.0) if norms[1] else None
        cos = sin = None
        if rope is not None:
            rows = batch * t if rope else t
            e = np.arange(rows * half)
            ang = (e // half).astype(np.float64) * 0.01 * (1.0 + (e % half).astype(np.float64))
            shape = (batch if rope else 1, t, 1, half)
            cos = oracle.round_bf16(np.cos(ang).astype(np.float32)).reshape(shape)
            sin = oracle.round_bf16(np.sin(ang).astype(np.float32)).reshape(shape)
        eps = rng.choice([1e-6, 1e-5])
        up = lambda a: None if a is None else bf16_tensor(a, device)
        name = f"case {case}: rows {batch}x{t} heads {hq}/{hk} d {d} norms {norms} rope {rope}"
        got = svod_amd.heads(up(qkv), Qkv(hq, hk, d, up(q_w), up(k_w), eps, None if cos is None else (up(cos), up(sin))))
        torch.cuda.synchronize()
        assert svod_amd.chosen().startswith('Kernel { op: "heads", family: "heads"'), (name, svod_amd.chosen())
        p = oracle.HeadsProblem(qkv, hq, hk, d, q_w, k_w, eps, cos, sin)
        direct, program = oracle.heads_direct(p), oracle.heads_kernel(p)
        for i, what in enumerate("qkv"):
            out = to_np(got[i])
            assert np.isfinite(out).all(), (name, what)
            assert max_abs(out, direct[i]) <= 2e-2, (name, what)   # heads.rs:124
            assert max_abs(out, program[i]) <= 1e-2, (name, what)  # heads.rs:159
        want_v = bf16_tensor(qkv.reshape(batch, t, slots, d)[:, :, hq + hk:, :], "cpu")
        assert np.array_equal(bits(got[2]), bits(want_v)), name
