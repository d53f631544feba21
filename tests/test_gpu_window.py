"""Sliding-window masks (Attn::window, tk/src/ops/attention.rs:64-65; tk/src/kernels/attention.rs:587-603,
659-668, 715-719) through the C ABI against the oracle.  The reference's own cases are the (20, 5) window
with key lengths and the (50, 0) one (tk/src/test/unit/attention.rs:280-289, 354); the longer ones are the
local attention of its ModernBERT layers (a window of 128 over a long sequence), where most key blocks
are skipped and the rest run the hot loop between two edges."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, assert_bf16_parity, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu


def case(b, t, tk, h, hkv, d, seed=5):
    g = Lcg(seed)
    return g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))


# (name, b, t, tk, h, hkv, d, window, causal, lens, splits)
CASES = [
    ("window with lengths", 2, 128, 128, 2, 2, 64, (20, 5), False, [128, 90], None),       # attention.rs:354
    ("a causal window", 2, 128, 128, 2, 2, 64, (50, 0), False, None, None),                 # attention.rs:289
    ("causal and a window that reaches ahead", 2, 200, 200, 2, 2, 64, (50, 7), True, None, None),
    ("local attention, 1024 tokens", 1, 1024, 1024, 4, 4, 64, (64, 64), False, None, None),
    ("local attention d 128, gqa, ragged", 2, 700, 700, 4, 2, 128, (128, 128), False, [700, 333], None),
    ("a window wider than the sequence", 2, 100, 100, 2, 2, 64, (500, 500), False, [100, 61], None),
    ("a window of the diagonal alone", 1, 130, 130, 2, 2, 64, (0, 0), False, None, None),
    ("a long look back, two splits", 1, 512, 512, 2, 2, 64, (300, 0), False, None, 2),
    ("cross lengths: more keys than queries", 1, 100, 400, 2, 2, 64, (30, 200), False, None, None),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,window,causal,lens,splits", CASES, ids=[c[0] for c in CASES])
def test_windowed_attention_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, d, window, causal, lens, splits):
    q, k, v = case(b, t, tk, h, hkv, d)
    keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                             Attn(causal=causal, keys=keys, window=window, splits=splits))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    got = to_np(got)
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=None if lens is None else np.asarray(lens), window=window)
    direct = oracle.attention_direct(p)
    program = oracle.attention_flash(p, bq=128, bkv=64, splits=splits or 1)
    assert_bf16_parity(name, got, direct, program)


def test_a_window_hides_exactly_its_complement(device):
    """One-hot values: out[i, c] is the softmax weight query i puts on key c, so it is zero exactly
    where the window (with the causal mask and the lengths) hides key c — bit for bit."""
    b, t, d, h = 2, 128, 64, 2
    g = Lcg(9)
    q, k = g.bf16((b, t, h, d)), g.bf16((b, t, h, d))
    for window, causal, lens in (((20, 5), False, [128, 90]), ((3, 0), True, None), ((0, 40), False, None)):
        for base in (0, 64):  # the keys whose weights the 64 value columns report
            v = np.zeros((b, t, h, d), dtype=np.float32)
            for c in range(d):
                v[:, base + c, :, c] = 1.0
            keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
            got = to_np(svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                                           Attn(causal=causal, keys=keys, window=window)))
            vis = oracle.visible(b, t, t, causal=causal, key_lens=lens, window=window)  # [B, T, Tk]
            want_zero = vis[:, :, base:base + d] == 0
            assert np.array_equal(got.transpose(0, 2, 1, 3)[:, 0] == 0, want_zero), (window, causal, base)
