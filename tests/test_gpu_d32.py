"""Head size 32 (tk/src/ops/shape.rs:189-206 with the configs of tk/src/ops/config/attention.rs:29-57: a head
size that tiles the matrix atom takes the kernel): the same kernel template at D = 32, against the oracle."""
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
    ("plain", 2, 130, 130, 4, 4, False, None, False, None, None, False),
    ("causal gqa, lengths", 3, 300, 300, 8, 2, True, [300, 129, 64], False, None, None, False),
    ("cross attention, bool mask", 2, 37, 500, 4, 4, False, None, True, None, None, False),
    ("a window", 1, 600, 600, 2, 2, False, None, False, (100, 20), None, False),
    ("three splits", 1, 64, 1000, 2, 2, False, [777], False, None, 3, False),
    ("biased causal", 2, 100, 100, 2, 1, True, None, False, None, None, True),
    ("long rows", 1, 1024, 1024, 2, 2, True, None, False, None, None, False),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,causal,lens,key_mask,window,splits,biased", CASES, ids=[c[0] for c in CASES])
def test_d32_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, causal, lens, key_mask, window, splits, biased):
    d = 32
    g = Lcg(5)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    bias = g.bf16((1, h, t, tk), mul=2.0) if biased else None
    mask = (np.add.outer(np.arange(b), np.arange(tk)) % 5 != 2) if key_mask else None
    keys = KeyMask.none()
    if lens is not None:
        keys = KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    if mask is not None:
        keys = KeyMask.bool(torch.from_numpy(mask).to(device))
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                             Attn(causal=causal, keys=keys, window=window, splits=splits or 1,
                                  bias=None if bias is None else bf16_tensor(bias, device)))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=None if lens is None else np.asarray(lens), key_mask=mask,
                           window=window, bias=bias)
    assert_bf16_parity(name, to_np(got), oracle.attention_direct(p), oracle.attention_flash(p, bq=128, bkv=64, splits=splits or 1))


def test_d32_f16_and_the_fused_projection(device):
    b, t, h, hkv, d = 2, 150, 4, 2, 32
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
