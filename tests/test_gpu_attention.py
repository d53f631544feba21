"""Parity of the HIP flash-attention forward (through the C ABI) with the CPU oracle.

Cases follow the reference's own: tk/src/test/unit/attention.rs:349-455
(``attention_matches_a_direct_softmax``; the mask forms this library has kernels for),
tk/src/test/unit/ops.rs:436-470 (``attention_matches_the_graph``), :1004-1024 (no-key rows)."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, assert_bf16_parity, assert_rel_close, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu


def reference_case(t, tk, d, heads=2, kv_heads=2, batch=2):
    """``case()`` of attention.rs:69-78: seed 5, q then k then v, uniform [-1,1) rounded to bf16."""
    g = Lcg(5)
    q = g.bf16((batch, t, heads, d))
    k = g.bf16((batch, tk, kv_heads, d))
    v = g.bf16((batch, tk, kv_heads, d))
    return q, k, v


def reference_key_mask(batch, tk):
    """Key j of batch b hidden where (b + j) % 5 == 2 (attention.rs:80-81)."""
    b, j = np.meshgrid(np.arange(batch), np.arange(tk), indexing="ij")
    return (b + j) % 5 != 2


def run(device, q, k, v, causal=False, lens=None, mask=None, scale=None, mask_dtype=torch.bool, lens_dtype=torch.int32,
        batch_live=None, out=None):
    keys = KeyMask.none()
    if lens is not None:
        keys = KeyMask.lens(torch.tensor(np.asarray(lens), dtype=lens_dtype, device=device))
    if mask is not None:
        keys = KeyMask.bool(torch.from_numpy(np.ascontiguousarray(mask)).to(mask_dtype).to(device))
    o = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                           Attn(causal=causal, keys=keys, scale=scale, batch_live=batch_live), out=out)
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention", family: "flash_attention"'), svod_amd.chosen()
    return o


# (name, t, tk, d, causal, lens, key_mask, scale)
DIRECT_CASES = [
    ("one block", 64, 64, 64, False, None, False, None),
    ("three key blocks", 128, 192, 64, False, None, False, None),
    ("causal", 128, 128, 64, True, None, False, None),
    ("key lengths", 128, 128, 64, False, [100, 7], False, None),
    ("causal with lengths", 128, 128, 64, True, [128, 50], False, None),
    ("key mask", 128, 128, 64, False, None, True, None),
    ("a lane with no keys", 128, 128, 64, False, [100, 0], False, None),
    ("causal, a lane with no keys", 128, 128, 64, True, [0, 50], False, None),
    ("a larger scale", 128, 128, 64, True, [128, 50], False, 0.3),
    ("a negative scale", 128, 128, 64, True, [128, 50], False, -0.1),
    ("plain", 128, 128, 64, False, None, False, None),
    ("causal, 256 queries", 256, 256, 64, True, None, False, None),
    ("key lengths, 256 keys", 128, 256, 64, False, [200, 33], False, None),
    ("d 128, causal with lengths", 128, 128, 128, True, [128, 64], False, None),
    ("bq 128, lens", 256, 192, 64, True, [192, 70], False, None),
    ("d 128, ragged", 200, 130, 128, False, [130, 99], False, None),
    ("d 128, bq 256, ragged", 600, 420, 128, False, [420, 299], False, None),
    ("key mask, ragged", 100, 100, 64, False, None, True, None),
    ("causal key mask with lengths, d 128", 128, 128, 128, True, [128, 100], True, None),
    ("ragged both ways", 99, 99, 64, False, [99, 41], False, None),
    ("one query row", 1, 200, 64, False, [200, 70], False, None),
]


@pytest.mark.parametrize("name,t,tk,d,causal,lens,key_mask,scale", DIRECT_CASES, ids=[c[0] for c in DIRECT_CASES])
def test_attention_matches_a_direct_softmax(device, name, t, tk, d, causal, lens, key_mask, scale):
    q, k, v = reference_case(t, tk, d)
    mask = reference_key_mask(2, tk) if key_mask else None
    # A kernel takes either mask form; both together only through lens folded into the mask.
    if mask is not None and lens is not None:
        mask = mask & (np.arange(tk)[None, :] < np.asarray(lens)[:, None])
        lens_arg = None
    else:
        lens_arg = lens
    got = to_np(run(device, q, k, v, causal, lens_arg, mask, scale))
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=None if lens_arg is None else np.asarray(lens_arg),
                           key_mask=mask, scale=scale)
    want = oracle.attention_direct(p)
    worst = max_abs(got, want)
    assert np.isfinite(got).all()
    assert worst < 2e-2, f"max abs diff {worst}"  # attention.rs:483
    # Against the tile program under the host interpreter at this kernel's tile: tighter.
    flash = oracle.attention_flash(p, bq=128, bkv=64)
    assert max_abs(got, flash) <= 1e-2  # attention.rs on_device_case


def graph_case(b, t, tk, h, hkv, d, seeds=(20, 21, 22)):
    """``attn_inputs`` of ops.rs:380-386 in spirit: three independent seeded tensors on [-1, 1)."""
    q = Lcg(seeds[0]).bf16((b, t, h, d))
    k = Lcg(seeds[1]).bf16((b, tk, hkv, d))
    v = Lcg(seeds[2]).bf16((b, tk, hkv, d))
    return q, k, v


GRAPH_CASES = [
    ("t100 key lens", 2, 100, 100, 4, 4, 64, False, [100, 61], False),
    ("causal t200", 1, 200, 200, 2, 2, 64, True, None, False),
    ("gqa 8 over 2", 2, 128, 128, 8, 2, 64, True, [128, 77], False),
    ("d128 gqa causal lens", 2, 100, 100, 4, 2, 128, True, [90, 100], False),
    ("cross attention", 2, 37, 150, 4, 4, 64, False, None, False),
    ("bool key mask", 2, 100, 100, 4, 4, 64, False, None, True),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,causal,lens,key_mask", GRAPH_CASES, ids=[c[0] for c in GRAPH_CASES])
def test_attention_matches_the_graph(device, name, b, t, tk, h, hkv, d, causal, lens, key_mask):
    q, k, v = graph_case(b, t, tk, h, hkv, d)
    mask = reference_key_mask(b, tk) if key_mask else None
    got = to_np(run(device, q, k, v, causal, lens, mask))
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=None if lens is None else np.asarray(lens), key_mask=mask)
    assert_rel_close("attention", got, oracle.attention_graph(p), 2e-2)  # ops.rs:464-469
    assert_bf16_parity(name, got, oracle.attention_direct(p), oracle.attention_flash(p, bq=128, bkv=64))


@pytest.mark.parametrize("by_lens", [True, False], ids=["a zero key length", "every key masked"])
def test_attention_to_no_key_is_zeros(device, by_lens):
    """ops.rs:1004-1024 and attention.rs:510-525: exact zeros, not NaN."""
    b, t, tk, h, d = 2, 64, 96, 4, 64
    q = Lcg(30).bf16((b, t, h, d))
    k = Lcg(31).bf16((b, tk, h, d))
    v = Lcg(32).bf16((b, tk, h, d))
    lens = [tk, 0] if by_lens else None
    mask = None if by_lens else (np.arange(b * tk) < tk).reshape(b, tk)
    got = to_np(run(device, q, k, v, False, lens, mask))
    assert np.isfinite(got).all()
    assert (got[1] == 0.0).all(), "the unreached batch is zeros"
    assert (got[0] != 0.0).any(), "the visible batch attends"
    p = oracle.AttnProblem(q, k, v, key_lens=None if lens is None else np.asarray(lens), key_mask=mask)
    assert_rel_close("attention to no key", got, oracle.attention_graph(p), 2e-2)


def test_only_the_live_batch_runs(device):
    """attention.rs:528-536: rows of a batch past the live bound are never written."""
    q, k, v = reference_case(64, 64, 64)
    out = torch.full((2, 64, 2, 64), float("nan"), dtype=torch.bfloat16, device=device)
    got = to_np(run(device, q, k, v, batch_live=1, out=out))
    assert np.isfinite(got[0]).all() and (got[0] != 0).any()
    assert np.isnan(got[1]).all(), "the batch past the live bound keeps its poison"


def test_lens_and_bool_masks_agree_bit_for_bit(device):
    """A right-padding Bool mask is the Lens mask: the two kernels' outputs are the same bits."""
    q, k, v = graph_case(3, 200, 200, 4, 2, 64)
    lens = np.array([200, 131, 64])
    mask = np.arange(200)[None, :] < lens[:, None]
    for causal in (False, True):
        a = run(device, q, k, v, causal, lens=lens)
        b8 = run(device, q, k, v, causal, mask=mask, mask_dtype=torch.bool)
        b32 = run(device, q, k, v, causal, mask=mask, mask_dtype=torch.int32)
        l64 = run(device, q, k, v, causal, lens=lens, lens_dtype=torch.int64)
        assert np.array_equal(bits(a), bits(b8))
        assert np.array_equal(bits(a), bits(b32))
        assert np.array_equal(bits(a), bits(l64))


def test_visibility_is_bit_exact(device):
    """With one-hot V rows (V[j] = e_j) the output row IS the softmax row: its zero pattern
    must equal the oracle's visibility predicate exactly, for every (b, i, j)."""
    b, t, tk, h, d = 2, 96, 64, 1, 64
    q = Lcg(3).bf16((b, t, h, d), mul=0.25)
    k = Lcg(4).bf16((b, tk, h, d), mul=0.25)
    v = np.zeros((b, tk, h, d), dtype=np.float32)
    for j in range(tk):
        v[:, j, :, j] = 1.0
    lens = np.array([64, 37])
    mask = reference_key_mask(b, tk) & (np.arange(tk)[None, :] < lens[:, None])
    for causal in (False, True):
        got = to_np(run(device, q, k, v, causal, mask=mask))[:, :, 0, :]  # [b, t, tk]
        vis = oracle.visible(b, t, tk, causal=causal, key_mask=mask).astype(bool)
        # Scores are O(1) here, so every visible key keeps a weight far above bf16's floor.
        assert np.array_equal(got != 0.0, vis)


MASK_PATTERNS = {
    "a hidden block in the middle, hidden blocks at the end": lambda b, tk: np.stack(
        [(np.arange(tk) < 300) & ~((np.arange(tk) >= 128) & (np.arange(tk) < 192)) for _ in range(b)]),
    "the first two blocks hidden": lambda b, tk: np.stack([np.arange(tk) >= 128 + 7 * i for i in range(b)]),
    "one visible key in the last block": lambda b, tk: np.stack([np.arange(tk) == tk - 1 - i for i in range(b)]),
    "every other block hidden": lambda b, tk: np.stack([(np.arange(tk) // 64 + i) % 2 == 0 for i in range(b)]),
    "a row of nothing": lambda b, tk: np.stack([np.zeros(tk, dtype=bool) if i == 1 else np.arange(tk) % 3 != 0 for i in range(b)]),
}


@pytest.mark.parametrize("pattern", list(MASK_PATTERNS), ids=list(MASK_PATTERNS))
@pytest.mark.parametrize("causal", [False, True])
def test_key_masks_with_whole_hidden_blocks(device, pattern, causal):
    """A key mask row is scanned at the start of a tile: blocks past its last visible key are skipped and
    leading blocks that hide nothing take the hot loop.  Whatever the pattern, the result is the direct softmax's,
    and the same as with the mask folded into an additive bias of -inf (which takes neither shortcut)."""
    b, t, tk, h, d = 3, 200, 500, 2, 64
    q, k, v = graph_case(b, t, tk, h, h, d)
    mask = MASK_PATTERNS[pattern](b, tk)
    got = to_np(run(device, q, k, v, causal, mask=mask))
    want = oracle.attention_direct(oracle.AttnProblem(q, k, v, causal=causal, key_mask=mask))
    assert max_abs(got, want) < 2e-2
    rows_without_keys = ~oracle.visible(b, t, tk, causal=causal, key_mask=mask).astype(bool).any(-1)  # [b, t]
    assert not got[rows_without_keys].any()
    walls = np.where(mask[:, None, None, :], 0.0, -np.inf).astype(np.float32) * np.ones((b, h, t, tk), dtype=np.float32)
    biased = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                                Attn(causal=causal, bias=bf16_tensor(np.nan_to_num(walls, nan=0.0, neginf=-np.inf), device)))
    assert max_abs(to_np(biased), want) < 2e-2


def test_a_key_mask_row_too_long_to_scan(device):
    """Past 256 blocks (16384 keys) the mask words are read two blocks ahead of their use instead."""
    b, t, tk, h, d = 1, 40, 16500, 1, 64
    q, k, v = graph_case(b, t, tk, h, h, d)
    mask = (np.arange(tk)[None, :] % 7 != 3) & (np.arange(tk)[None, :] < 16450)
    keys = KeyMask.bool(torch.from_numpy(mask).to(device))
    want = oracle.attention_direct(oracle.AttnProblem(q, k, v, key_mask=mask))
    dq, dk, dv = (bf16_tensor(x, device) for x in (q, k, v))
    whole = svod_amd.attention(dq, dk, dv, Attn(keys=keys, splits=1))  # one pass over 258 blocks: too long to scan
    assert "flash_attention" in svod_amd.chosen()
    assert max_abs(to_np(whole), want) < 2e-2
    split = svod_amd.attention(dq, dk, dv, Attn(keys=keys))  # split unasked: every split scans its share
    assert "combine_splits" in svod_amd.chosen()
    assert max_abs(to_np(split), want) < 2e-2


@pytest.mark.parametrize("per_key,causal,d", [(0.1, False, 64), (1.0, False, 64), (0.1, True, 64), (0.4, False, 128),
                                               (-0.5, False, 64)],
                         ids=["a slow climb", "a steep climb", "a slow causal climb", "d 128", "a descent"])
def test_climbing_scores_rescale_the_accumulator(device, per_key, causal, d):
    """attention.rs:457-472 with the climb in the scores themselves (its bias-ramp form is in
    test_gpu_bias.py): key j scores per_key * j in log2 units against every query, so a row keeps its
    stale maximum for several blocks and then adopts a new one (slowly), or adopts one every block
    (steeply); the accumulator is rescaled while it holds earlier blocks' work.  A descent never rescales."""
    b, t, tk, h = 2, 256, 512, 2
    g = Lcg(5)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, h, d)), g.bf16((b, tk, h, d))
    # One coordinate carries the ramp: q[..., 0] = 1, k[j, ..., 0] = ramp(j); the others stay small noise.
    q[..., 0] = 1.0
    ramp = oracle.round_bf16((per_key * np.arange(tk) / (d ** -0.5 * 1.4426950408889634)).astype(np.float32))
    k[..., 0] = ramp[None, :, None]
    q[..., 1:] *= 0.25
    lens = [tk, 300]
    got = to_np(run(device, q, k, v, causal=causal, lens=lens))
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=np.asarray(lens))
    assert_bf16_parity("climbing scores", got, oracle.attention_direct(p), oracle.attention_flash(p, bq=128, bkv=64))


def test_a_non_finite_unread_element_never_reaches_the_output(device):
    """attention.rs:572-592 on plain operands: rows of K and V at and past a batch row's length may
    hold anything, an infinity or a NaN included, as memory nothing initialised does; the kernel reads
    zeros there (the last key block is partial), never those elements."""
    b, t, tk, h, d = 2, 100, 200, 4, 64
    q, k, v = reference_case(t, tk, d, heads=h, kv_heads=h, batch=b)
    lens = [100, 37]
    clean = run(device, q, k, v, lens=lens)
    for x in (k, v):
        x[0, 100:] = np.nan
        x[1, 37:] = np.inf
        x[1, 38::2] = np.nan
    dirty = run(device, q, k, v, lens=lens)
    assert np.isfinite(to_np(dirty)).all()
    assert np.array_equal(bits(dirty), bits(clean))
    for causal in (True,):
        assert np.isfinite(to_np(run(device, q, k, v, causal=causal, lens=lens))).all()
