"""Head size 256 (tk/src/ops/shape.rs:189-206 and the reference's plan test tk/src/test/unit/ops_plan.rs:1241-1262:
256 tiles the matrix atom and takes the kernel): the same kernel template at D = 256 (a 128 KiB ring, one wave a
SIMD), against the oracle, over the mask forms, splits, a cache and both 16-bit types."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, Cache, KeyMask
from util import Lcg, assert_bf16_parity, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu
D = 256

# (name, b, t, tk, h, hkv, causal, lens, key_mask, window, splits, biased)
CASES = [
    ("one block", 1, 64, 64, 1, 1, False, None, False, None, None, False),
    ("plain, ragged", 2, 130, 130, 2, 2, False, None, False, None, None, False),
    ("causal gqa, lengths", 3, 300, 300, 4, 2, True, [300, 129, 64], False, None, None, False),
    ("cross attention, bool mask", 2, 37, 500, 2, 2, False, None, True, None, None, False),
    ("a window", 1, 400, 400, 2, 2, False, None, False, (100, 20), None, False),
    ("three splits", 1, 64, 1000, 2, 2, False, [777], False, None, 3, False),
    ("biased causal", 2, 100, 100, 2, 1, True, None, False, None, None, True),
    ("long rows: the hot loop", 1, 1024, 1024, 2, 1, True, None, False, None, None, False),
    ("a lane with no keys", 2, 128, 128, 2, 2, False, [100, 0], False, None, None, False),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,causal,lens,key_mask,window,splits,biased", CASES, ids=[c[0] for c in CASES])
def test_d256_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, causal, lens, key_mask, window, splits, biased):
    g = Lcg(5)
    q, k, v = g.bf16((b, t, h, D)), g.bf16((b, tk, hkv, D)), g.bf16((b, tk, hkv, D))
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


def test_d256_visibility_is_bit_exact(device):
    """One-hot values: the output row is the set of keys a query saw, so a wrong mask bit shows as a wrong bit."""
    b, t, tk, h = 1, 200, 256, 1
    q = np.zeros((b, t, h, D), dtype=np.float32)  # equal scores: every visible key weighs the same
    k = Lcg(7).bf16((b, tk, h, D))
    v = np.zeros((b, tk, h, D), dtype=np.float32)
    v[0, np.arange(tk), 0, np.arange(tk)] = 1.0
    lens = [190]
    got = to_np(svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                                   Attn(causal=True, keys=KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device)))))
    torch.cuda.synchronize()
    seen = got[0, :, 0, :] > 0
    want = oracle.visible(b, t, tk, causal=True, key_lens=np.asarray(lens))[0]
    assert np.array_equal(seen, np.asarray(want, dtype=bool)[:, :D])


def test_d256_f16_and_the_fused_projection(device):
    b, t, h, hkv = 2, 150, 2, 1
    x = torch.from_numpy(oracle.round_f16(Lcg(3).bf16((b, t, (h + 2 * hkv) * D)))).to(torch.float16).to(device)
    packed = svod_amd.attention_packed(x, h, hkv, Attn(causal=True))
    q, k, v = x.view(b, t, h + 2 * hkv, D).split([h, hkv, hkv], dim=2)
    split = svod_amd.attention(q.contiguous(), k.contiguous(), v.contiguous(), Attn(causal=True))
    torch.cuda.synchronize()
    a, c = (y.detach().cpu().view(torch.int16).numpy() for y in (packed, split))
    assert np.array_equal(a, c)
    f = lambda y: y.detach().cpu().to(torch.float32).numpy()
    want = oracle.attention_direct(oracle.AttnProblem(f(q), f(k), f(v), causal=True))
    assert max_abs(f(split), want) < 2e-2


def test_d256_decoder_step_over_a_cache(device):
    """A grouped GQA decoder step over a cache that holds two layers' heads, keys split by the library."""
    b, tk, h, hkv, layers = 2, 700, 4, 2, 2
    g = Lcg(11)
    q = g.bf16((b, 1, h, D))
    kc, vc = g.bf16((b, tk, layers * hkv, D)), g.bf16((b, tk, layers * hkv, D))
    lens = np.array([700, 333])
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(kc, device), bf16_tensor(vc, device),
                             Attn(keys=KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device)), cache=Cache(hkv, hkv)))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, kc[:, :, hkv:2 * hkv], vc[:, :, hkv:2 * hkv], key_lens=lens)
    assert max_abs(to_np(got), oracle.attention_direct(p)) < 2e-2
