"""Chunk masks and segment starts (Attn::chunk, Attn::seg_start: tk/src/ops/attention.rs:39-50, 66-71;
tk/src/kernels/attention.rs:573-606, 669-695, 720-731) through the C ABI against the oracle.  The first
cases are the reference's own (tk/src/test/unit/attention.rs:282-294, 356-358; tk/src/test/unit/ops.rs:
398-401, 444-445, 452-454) at the head sizes this library has kernels for; the longer ones put several
hot blocks between a range's two edges and cross tiles, heads and splits."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, assert_bf16_parity, bf16_tensor, bits, to_np

pytestmark = pytest.mark.gpu


def case(b, t, tk, h, hkv, d, seed=5):
    g = Lcg(seed)
    return g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))


def segments(b, t, length):
    """Rows packed in segments of `length`: x % t - x % t % length (attention.rs:81, ops.rs:399)."""
    return np.tile(np.arange(t) - np.arange(t) % length, (b, 1))


def key_mask_of(b, tk):
    return np.add.outer(np.arange(b), np.arange(tk)) % 5 != 2  # attention.rs:80


# (name, b, t, tk, h, hkv, d, masks, lens, splits); masks: causal, window, chunk, segment length, key_mask
CASES = [
    ("causal segments", 2, 128, 128, 2, 2, 64, dict(causal=True, seg=40), None, None),                 # attention.rs:356
    ("chunks with lengths", 2, 128, 128, 2, 2, 64, dict(chunk=(16, 2, 0)), [128, 90], None),             # attention.rs:357
    ("chunks, every earlier one and one ahead, ragged", 2, 100, 100, 2, 2, 64, dict(chunk=(24, None, 1)), None, None),
    ("every mask at once", 2, 128, 128, 2, 2, 64,
     dict(causal=True, window=(50, 0), chunk=(32, 3, 0), seg=40, key_mask=True), [128, 100], None),      # attention.rs:288-295
    ("causal packed segments, gqa", 2, 200, 200, 4, 2, 64, dict(causal=True, seg=30), None, None),       # ops.rs:444
    ("chunks of 8, sixteen behind, lens", 2, 300, 300, 4, 4, 64, dict(chunk=(8, 16, 0)), [300, 171], None),  # ops.rs:452
    ("d48 chunks of 8, sixteen behind, lens", 2, 300, 300, 4, 4, 48, dict(chunk=(8, 16, 0)), [300, 171], None),  # ops.rs:452
    ("d48 causal segments bool mask", 1, 96, 96, 4, 4, 48, dict(causal=True, seg=40, key_mask=True), None, None),  # ops.rs:445
    ("chunks of 24, every earlier one and one ahead", 2, 200, 200, 4, 2, 64, dict(chunk=(24, None, 1)), None, None),
    ("d128 chunks with a bool mask", 1, 100, 100, 4, 4, 128, dict(chunk=(16, 1, 0), key_mask=True), None, None),
    ("long segments, d128", 1, 900, 900, 2, 1, 128, dict(causal=True, seg=333), None, None),
    ("segments without a causal mask", 2, 500, 500, 2, 2, 64, dict(seg=170), [500, 444], None),
    ("wide chunks over 1024 tokens", 1, 1024, 1024, 2, 2, 64, dict(chunk=(200, 1, 0)), None, None),
    ("chunks that see only themselves", 1, 640, 640, 2, 2, 64, dict(chunk=(128, 0, 0)), None, None),
    ("chunks ahead only, two splits", 1, 512, 512, 2, 2, 64, dict(chunk=(64, 0, 3)), None, 2),
    ("segments, three splits", 1, 600, 600, 2, 2, 64, dict(causal=True, seg=250), None, 3),
    ("more keys than queries", 1, 100, 400, 2, 2, 64, dict(chunk=(50, 1, 2)), None, None),
]


def run(device, b, t, tk, h, hkv, d, masks, lens, splits, seg_dtype=torch.int32):
    q, k, v = case(b, t, tk, h, hkv, d)
    masks = dict(masks)
    seg = segments(b, t, masks.pop("seg")) if "seg" in masks else None
    key_mask = key_mask_of(b, tk) if masks.pop("key_mask", False) else None
    if key_mask is not None and lens is not None:
        key_mask = key_mask & (np.arange(tk)[None, :] < np.asarray(lens)[:, None])  # one KeyMask a call: lengths folded in
        keys = KeyMask.bool(torch.from_numpy(key_mask).to(device))
    elif key_mask is not None:
        keys = KeyMask.bool(torch.from_numpy(key_mask).to(device))
    elif lens is not None:
        keys = KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    else:
        keys = KeyMask.none()
    seg_t = None if seg is None else torch.from_numpy(seg).to(seg_dtype).to(device)
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                             Attn(keys=keys, seg_start=seg_t, splits=splits, **masks))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, k, v, key_lens=None if (lens is None or key_mask is not None) else np.asarray(lens),
                           key_mask=key_mask, seg_start=seg, **masks)
    return got, p


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,masks,lens,splits", CASES, ids=[c[0] for c in CASES])
def test_ranged_attention_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, d, masks, lens, splits):
    got, p = run(device, b, t, tk, h, hkv, d, masks, lens, splits)
    direct = oracle.attention_direct(p)
    program = oracle.attention_flash(p, bq=128, bkv=64, splits=splits or 1)
    assert_bf16_parity(name, to_np(got), direct, program)


def test_segment_starts_may_be_64_bit(device):
    a, _ = run(device, 2, 200, 200, 4, 2, 64, dict(causal=True, seg=30), None, None, seg_dtype=torch.int32)
    b, _ = run(device, 2, 200, 200, 4, 2, 64, dict(causal=True, seg=30), None, None, seg_dtype=torch.int64)
    assert np.array_equal(bits(a), bits(b))


@pytest.mark.parametrize("masks,lens", [(dict(chunk=(16, 2, 0)), [128, 90]), (dict(chunk=(24, None, 1)), None),
                                        (dict(causal=True, seg=40), None), (dict(seg=50, chunk=(32, None, 0)), [100, 128])],
                         ids=["chunks behind", "chunks ahead", "causal segments", "segments and chunks"])
def test_a_range_hides_exactly_its_complement(device, masks, lens):
    """One-hot values: out[i, c] is the softmax weight query i puts on key c, so it is zero exactly
    where the masks hide key c — bit for bit."""
    b, t, d, h = 2, 128, 64, 2
    g = Lcg(9)
    q, k = g.bf16((b, t, h, d)), g.bf16((b, t, h, d))
    masks = dict(masks)
    seg = segments(b, t, masks.pop("seg")) if "seg" in masks else None
    keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    seg_t = None if seg is None else torch.from_numpy(seg).to(torch.int32).to(device)
    for base in (0, 64):  # the keys whose weights the 64 value columns report
        v = np.zeros((b, t, h, d), dtype=np.float32)
        for c in range(d):
            v[:, base + c, :, c] = 1.0
        got = to_np(svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                                       Attn(keys=keys, seg_start=seg_t, **masks)))
        vis = oracle.visible(b, t, t, key_lens=lens, seg_start=seg, **masks)  # [B, T, Tk]
        want_zero = vis[:, :, base:base + d] == 0
        assert np.array_equal(got.transpose(0, 2, 1, 3)[:, 0] == 0, want_zero), base


def test_masks_that_are_other_masks_agree_bit_for_bit(device):
    """A chunk mask of size 1 is a window; one chunk over everything and segments from key 0 hide nothing."""
    b, t, h, d = 2, 300, 2, 64
    q, k, v = (bf16_tensor(x, device) for x in case(b, t, t, h, h, d))
    plain = bits(svod_amd.attention(q, k, v))
    assert np.array_equal(bits(svod_amd.attention(q, k, v, Attn(chunk=(t, 0, 0)))), plain)
    zeros = torch.zeros((b, t), dtype=torch.int32, device=device)
    assert np.array_equal(bits(svod_amd.attention(q, k, v, Attn(seg_start=zeros))), plain)
    assert np.array_equal(bits(svod_amd.attention(q, k, v, Attn(chunk=(1, 20, 5)))),
                          bits(svod_amd.attention(q, k, v, Attn(window=(20, 5)))))
    assert np.array_equal(bits(svod_amd.attention(q, k, v, Attn(chunk=(1, None, 0)))),
                          bits(svod_amd.attention(q, k, v, Attn(causal=True))))
