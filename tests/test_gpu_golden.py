"""The HIP kernels against the committed golden fixtures (expected values from torch float64
SDPA / numpy float64, see tests/golden/make_golden.py) and at the benchmark's own shapes."""
import glob
import os

import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, Fallback, GraphFallback, KeyMask, Qkv, workloads as W
from util import assert_bf16_parity, bf16_tensor, bits, max_abs, mean_rel, to_np

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
ATTN = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "attn_*.npz")))
HEADS = sorted(os.path.basename(p)[:-4] for p in glob.glob(os.path.join(GOLDEN, "heads_*.npz")))


def load(name):
    return dict(np.load(os.path.join(GOLDEN, name + ".npz")))


@pytest.mark.parametrize("name", ATTN)
def test_attention_fixture(device, name):
    g = load(name)
    keys = KeyMask.none()
    if "lens" in g:
        keys = KeyMask.lens(torch.from_numpy(g["lens"]).to(device))
    if "key_mask" in g:
        keys = KeyMask.bool(torch.from_numpy(g["key_mask"]).to(device))
    o = svod_amd.attention(bf16_tensor(g["q"], device), bf16_tensor(g["k"], device), bf16_tensor(g["v"], device),
                           Attn(causal=bool(g["causal"]), keys=keys, scale=float(g["scale"])))
    got = to_np(o)
    assert np.isfinite(got).all()
    assert max_abs(got, g["out"]) < 2e-2
    none = ~g["keep"].any(axis=-1)  # [B, T] rows no key reaches
    assert (got[none] == 0.0).all()


@pytest.mark.parametrize("name", HEADS)
def test_heads_fixture(device, name):
    g = load(name)
    h, hkv, d = (int(x) for x in g["dims"])
    t = g["cos"].shape[0]
    tb = lambda a: bf16_tensor(a, device)
    q, k, v = svod_amd.heads(tb(g["qkv"]), Qkv(h, hkv, d, tb(g["q_w"]), tb(g["k_w"]), float(g["eps"]),
                                               (tb(g["cos"].reshape(1, t, 1, d // 2)), tb(g["sin"].reshape(1, t, 1, d // 2)))))
    for got, what in ((q, "q"), (k, "k"), (v, "v")):
        assert max_abs(to_np(got), g[what]) <= 2e-2, what
    assert np.array_equal(to_np(v), g["v"].astype(np.float32))


def test_config1_fp32_keeps_the_graph_and_its_bf16_cast_runs(device):
    """Config 1 is fp32: the op layer sends f32 to the graph (tk/src/ops/shape.rs:92-99), as the
    reference does.  The same inputs cast to bf16 take the kernel and agree with the oracle."""
    g = load("config1_fp32")
    q, k, v = (torch.from_numpy(g[n]).to(device) for n in "qkv")
    with pytest.raises(GraphFallback) as e:
        svod_amd.attention(q, k, v, Attn(scale=0.125))
    assert e.value.why == Fallback.Dtype
    assert svod_amd.chosen() == 'Graph { op: "attention", why: Dtype }'
    qb, kb, vb = (x.to(torch.bfloat16) for x in (q, k, v))
    got = to_np(svod_amd.attention(qb, kb, vb, Attn(scale=0.125)))
    p = oracle.AttnProblem(to_np(qb), to_np(kb), to_np(vb), scale=0.125)
    assert_bf16_parity("config 1 in bf16", got, oracle.attention_direct(p), oracle.attention_flash(p, 128, 64))
    # bf16 inputs against the fp32 problem's float64 answer: input rounding dominates.
    assert max_abs(got, g["out"]) < 2e-2


def sample_slices(w, picks):
    """Sub-problems (one batch row, one KV group) of a workload for the oracle."""
    b, t, tk, h, hkv, d = w.dims
    group = h // hkv
    for bi, kvh in picks:
        hs = slice(kvh * group, (kvh + 1) * group)
        lens = None if w.key_lens is None else w.key_lens[bi:bi + 1].cpu().numpy()
        yield bi, hs, oracle.AttnProblem(to_np(w.q[bi:bi + 1, :, hs]), to_np(w.k[bi:bi + 1, :, kvh:kvh + 1]),
                                         to_np(w.v[bi:bi + 1, :, kvh:kvh + 1]), causal=w.causal, key_lens=lens,
                                         scale=w.scale)


def torch_attention_everywhere(w, o):
    """Every element of `o` against matmul -> mask -> softmax -> matmul in f32 with plain torch ops on
    the device (the routine the golden fixtures are made with, tests/golden/make_golden.py, here in f32
    and one (batch row, head) chunk at a time so that the scores of an 8192-key row fit).  Returns the
    worst absolute difference over the whole tensor."""
    b, t, tk, h, hkv, d = w.dims
    group = h // hkv
    scale = w.scale if w.scale is not None else d ** -0.5
    rows = torch.arange(t, device=o.device).unsqueeze(1)
    cols = torch.arange(tk, device=o.device).unsqueeze(0)
    heads_a_chunk = max(1, min(h, (1 << 28) // max(1, t * tk)))  # at most 1 GiB of f32 scores at a time
    worst = 0.0
    for bi in range(b):
        keep = torch.ones((t, tk), dtype=torch.bool, device=o.device)
        if w.key_lens is not None:
            keep &= cols < int(w.key_lens[bi])
        if w.causal:
            keep &= cols <= rows
        for h0 in range(0, h, heads_a_chunk):
            hs = torch.arange(h0, min(h, h0 + heads_a_chunk), device=o.device)
            q = w.q[bi, :, hs].float().transpose(0, 1)                 # [heads, T, D]
            k = w.k[bi][:, hs // group].float().transpose(0, 1)        # [heads, Tk, D]
            v = w.v[bi][:, hs // group].float().transpose(0, 1)
            s = torch.matmul(q, k.transpose(1, 2)) * scale
            s = s.masked_fill(~keep, float("-inf"))
            p = torch.softmax(s, dim=-1)
            p = torch.where(keep.any(dim=1, keepdim=True), p, torch.zeros_like(p))  # a row no key reaches: zeros
            want = torch.matmul(p, v).transpose(0, 1)                  # [T, heads, D]
            worst = max(worst, float((o[bi, :, hs].float() - want).abs().max()))
            del s, p, want
    return worst


def check_workload(device, w, picks, bool_mask=False, everywhere=True):
    keys = KeyMask.none()
    if w.key_lens is not None:
        keys = KeyMask.bool(w.key_mask()) if bool_mask else KeyMask.lens(w.key_lens)
    out = torch.full_like(w.q, float("nan"))
    o = svod_amd.attention(w.q, w.k, w.v, Attn(causal=w.causal, keys=keys, scale=w.scale), out=out)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all(), "an element was left unwritten or is not finite"
    for bi, hs, p in sample_slices(w, picks):
        got = to_np(o[bi:bi + 1, :, hs])
        assert_bf16_parity(f"{w.name} b{bi} h{hs}", got, oracle.attention_direct(p), oracle.attention_flash(p, 128, 64))
    if everywhere:
        worst = torch_attention_everywhere(w, o)
        assert worst <= 2e-2, f"{w.name}: max-abs {worst} over the whole tensor"  # tk/src/test/unit/attention.rs:483
    return o


def test_config2_bge_m3_full_size(device):
    w = W.config2(layer=0, device=device)
    lens = w.key_lens.tolist()
    picks = [(int(np.argmin(lens)), 0), (int(np.argmax(lens)), 15), (7, 3)]
    o = check_workload(device, w, picks)
    ob = check_workload(device, w, picks[:1], bool_mask=True, everywhere=False)  # the same bits, asserted below
    assert torch.equal(o.view(torch.int16), ob.view(torch.int16)), "Lens and Bool masks give the same bits"
    # Size-independent property: keys past the length do not matter.  Poison them and rerun.
    k2, v2 = w.k.clone(), w.v.clone()
    pad = ~w.key_mask()
    k2[pad] = float("nan")
    v2[pad] = 1e30
    o2 = svod_amd.attention(w.q, k2, v2, Attn(keys=KeyMask.lens(w.key_lens), scale=w.scale))
    assert torch.equal(o.view(torch.int16), o2.view(torch.int16))


def test_config3_qwen3_prologue_and_attention_full_size(device):
    p = W.config3_prologue(device=device)
    q, k, v = svod_amd.heads(p.qkv, Qkv(p.heads, p.kv_heads, p.head_dim, p.q_w, p.k_w, p.eps, (p.cos, p.sin)))
    torch.cuda.synchronize()
    # Prologue parity on sampled rows (first, last and two inside) against the oracle.
    rows = [0, 1, 777, 2047]
    for bi in (0, 7):
        sub = oracle.HeadsProblem(to_np(p.qkv[bi:bi + 1, rows]), p.heads, p.kv_heads, p.head_dim, to_np(p.q_w),
                                  to_np(p.k_w), p.eps, to_np(p.cos[0, rows, 0]), to_np(p.sin[0, rows, 0]))
        want = oracle.heads_direct(sub)
        prog = oracle.heads_kernel(sub)
        for got, wd, wp, what in zip((q, k, v), want, prog, "qkv"):
            g = to_np(got[bi:bi + 1, rows])
            assert max_abs(g, wd) <= 2e-2 and max_abs(g, wp) <= 1e-2, what
    # Every element of q and k against the same arithmetic in f32 with plain torch ops on the device
    # (tk/src/kernels/heads.rs:73-111), at the op-against-graph bar of tk/src/test/unit/mod.rs:526-536.
    x = p.qkv.view(8, 2048, 32, 128).float()
    cos, sin = p.cos.float(), p.sin.float()  # [1, T, 1, D/2]
    for got, sl, wn, what in ((q, slice(0, 16), p.q_w, "q"), (k, slice(16, 24), p.k_w, "k")):
        xs = x[:, :, sl]
        y = xs * torch.rsqrt((xs * xs).mean(dim=-1, keepdim=True) + p.eps) * wn.float()
        y1, y2 = y[..., :64], y[..., 64:]
        want = torch.cat((y1 * cos - y2 * sin, y1 * sin + y2 * cos), dim=-1)
        diff = (got.float() - want).abs()
        assert bool((diff <= 2e-2 * want.abs().clamp(min=1.0)).all()), f"{what}: worst {float(diff.max())} over the whole tensor"
        del xs, y, want, diff
    del x
    # v is the input's v slots bit for bit, everywhere.
    vin = p.qkv.view(8, 2048, 32, 128)[:, :, 24:, :]
    assert torch.equal(v.view(torch.int16), vin.contiguous().view(torch.int16))
    w = W.config3_attention(q, k, v)
    lens = w.key_lens.tolist()
    picks = [(int(np.argmin(lens)), 0), (int(np.argmax(lens)), 7)]
    check_workload(device, w, picks)


def test_config4_whisper_full_size(device):
    w = W.config4(device=device)
    check_workload(device, w, [(0, 0), (15, 19)])


def test_config5_long_context_full_size(device):
    w = W.config5(device=device)
    o = check_workload(device, w, [(1, 3)])
    # Linearity in V: attention(q, k, a·v) = a·attention(q, k, v) for a power of two, bit for bit.
    o2 = svod_amd.attention(w.q, w.k, (w.v.float() * 4.0).to(torch.bfloat16),
                            Attn(keys=KeyMask.lens(w.key_lens), scale=w.scale))
    assert torch.equal((o.float() * 4.0).to(torch.bfloat16).view(torch.int16), o2.view(torch.int16))


def test_permuting_keys_with_their_values_changes_nothing_beyond_rounding(device):
    """Softmax attention is invariant to a permutation of (key, value) pairs.  The two runs round
    their bf16 probabilities against different running maxima, so each carries its own
    ~1.6e-3 of probability-rounding noise; they agree to within twice that."""
    w = W.config2(layer=1, batch=4, seq=512, device=device)
    perm = torch.randperm(512, generator=torch.Generator().manual_seed(0)).to(device)
    mask = w.key_mask()
    a = svod_amd.attention(w.q, w.k, w.v, Attn(keys=KeyMask.bool(mask), scale=w.scale))
    b = svod_amd.attention(w.q, w.k[:, perm].contiguous(), w.v[:, perm].contiguous(),
                           Attn(keys=KeyMask.bool(mask[:, perm].contiguous()), scale=w.scale))
    assert mean_rel(to_np(b), to_np(a)) < 4e-3
    assert max_abs(to_np(b), to_np(a)) < 1e-2
