"""Head size 48 (tk/src/ops/shape.rs:189-206: a head size that tiles the matrix atom takes the kernel; the
reference's own d 48 cases are tk/src/test/unit/ops.rs:445-446,452,589-590 and attention.rs:360,402-404,430-431).
The kernel runs it on the 64-wide tile: a row's last two 16-byte chunks are never fetched, the score product
stops at the third k-step, the tile's columns past the head are dropped at the store.  The cases with a cache are
in test_gpu_cache.py, those with chunks and segments in test_gpu_ranges.py."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, assert_bf16_parity, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu

# (name, b, t, tk, h, hkv, causal, lens, key_mask, window, splits, biased)
CASES = [
    ("d48 key lens", 2, 150, 150, 4, 4, False, [150, 100], False, None, None, False),  # ops.rs:446
    ("d 48, 96 queries", 1, 96, 96, 4, 4, False, None, False, None, None, False),     # attention.rs:360
    ("d 48, 200 queries causal", 1, 200, 200, 2, 2, True, None, False, None, None, False),  # attention.rs:430
    ("causal gqa, lengths", 3, 300, 300, 8, 2, True, [300, 129, 64], False, None, None, False),
    ("cross attention, bool mask", 2, 37, 500, 4, 4, False, None, True, None, None, False),
    ("a window", 1, 600, 600, 2, 2, False, None, False, (100, 20), None, False),
    ("three splits", 1, 64, 1000, 2, 2, False, [777], False, None, 3, False),
    ("biased causal", 2, 100, 100, 2, 1, True, None, False, None, None, True),
    ("long rows", 1, 1024, 1024, 2, 2, True, None, False, None, None, False),
    ("one query, a decoder step split by the rule", 4, 1, 3000, 8, 2, False, [3000, 2999, 64, 1], False, None, 0, False),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,causal,lens,key_mask,window,splits,biased", CASES, ids=[c[0] for c in CASES])
def test_d48_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, causal, lens, key_mask, window, splits, biased):
    d = 48
    g = Lcg(5)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    bias = g.bf16((1, h, t, tk), mul=2.0) if biased else None
    mask = (np.add.outer(np.arange(b), np.arange(tk)) % 5 != 2) if key_mask else None
    keys = KeyMask.none()
    if lens is not None:
        keys = KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    if mask is not None:
        keys = KeyMask.bool(torch.from_numpy(mask).to(device))
    out = torch.full((b, t, h, d), 7.0, dtype=torch.bfloat16, device=device)
    guard = torch.full((b * t * h * d + 64,), 7.0, dtype=torch.bfloat16, device=device)  # out, and 64 elements behind it
    out = guard[:b * t * h * d].view(b, t, h, d)
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                             Attn(causal=causal, keys=keys, window=window, splits=1 if splits is None else splits,
                                  bias=None if bias is None else bf16_tensor(bias, device)), out=out)
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    assert (guard[b * t * h * d:].float() == 7.0).all(), "the tile's columns past the head were stored"
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=None if lens is None else np.asarray(lens), key_mask=mask,
                           window=window, bias=bias)
    direct = oracle.attention_direct(p)
    if splits == 0:  # the rule's own count: held to the direct softmax
        assert "combine_splits" in svod_amd.chosen()
        assert max_abs(to_np(got), direct) < 2e-2
        return
    assert_bf16_parity(name, to_np(got), direct, oracle.attention_flash(p, bq=128, bkv=64, splits=splits or 1))


def test_d48_equals_d64_with_zero_columns(device):
    """Padding every head with 16 zero columns changes no score and adds zero output columns: with the
    scale held, the 64-wide call's first 48 columns are the 48-wide call's, bit for bit."""
    b, t, h, hkv = 2, 200, 4, 2
    g = Lcg(11)
    q, k, v = g.bf16((b, t, h, 48)), g.bf16((b, t, hkv, 48)), g.bf16((b, t, hkv, 48))
    pad = lambda x: np.concatenate([x, np.zeros(x.shape[:-1] + (16,), dtype=x.dtype)], axis=-1)
    lens = torch.tensor([200, 77], dtype=torch.int32, device=device)
    opts = Attn(causal=True, keys=KeyMask.lens(lens), scale=48 ** -0.5)
    narrow = svod_amd.attention(*(bf16_tensor(x, device) for x in (q, k, v)), opts)
    wide = svod_amd.attention(*(bf16_tensor(pad(x), device) for x in (q, k, v)), opts)
    torch.cuda.synchronize()
    assert np.array_equal(bits(narrow), bits(wide[..., :48].contiguous()))
    assert not bits(wide[..., 48:].contiguous()).any()


def test_d48_f16_and_the_fused_projection(device):
    b, t, h, hkv, d = 2, 150, 4, 2, 48
    x = torch.from_numpy(oracle.round_f16(Lcg(3).bf16((b, t, (h + 2 * hkv) * d)))).to(torch.float16).to(device)
    packed = svod_amd.attention_packed(x, h, hkv, Attn(causal=True))
    q, k, v = x.view(b, t, h + 2 * hkv, d).split([h, hkv, hkv], dim=2)
    split = svod_amd.attention(q.contiguous(), k.contiguous(), v.contiguous(), Attn(causal=True))
    torch.cuda.synchronize()
    a, c = (y.detach().cpu().view(torch.int16).numpy() for y in (packed, split))
    assert np.array_equal(a, c)
    f = lambda y: y.detach().cpu().to(torch.float32).numpy()
    want = oracle.attention_direct(oracle.AttnProblem(f(q), f(k), f(v), causal=True))
    assert max_abs(f(split), want) < 2e-2
