"""The f16 instantiations (through the C ABI) against the oracle rounding to f16: the reference's
kernels run either 16-bit float type (tk/src/ops/shape.rs:92-99, tk/src/build.rs:50-64); the cases
are a sample of the bf16 ones (tk/src/test/unit/attention.rs:349-455, heads.rs:112-161)."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask, Qkv
from util import Lcg, max_abs, mean_rel, to_np

pytestmark = pytest.mark.gpu


def f16_tensor(a, device):
    """f16-exact float32 values as an f16 tensor (the cast is exact)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.float16).to(device)


def f16_bits(t):
    return t.detach().to("cpu").view(torch.int16).numpy().view(np.uint16)


def case(t, tk, d, heads=2, kv_heads=2, batch=2, seed=5):
    g = Lcg(seed)
    mk = lambda shape: oracle.round_f16(g.bf16(shape))  # bf16-exact values are f16-exact in [-1, 1) down to 2^-14
    return mk((batch, t, heads, d)), mk((batch, tk, kv_heads, d)), mk((batch, tk, kv_heads, d))


# (name, t, tk, d, heads, kv_heads, causal, lens, key_mask, scale, splits)
CASES = [
    ("three key blocks", 128, 192, 64, 2, 2, False, None, False, None, None),
    ("causal with lengths", 128, 128, 64, 2, 2, True, [128, 50], False, None, None),
    ("key mask, ragged", 100, 100, 64, 2, 2, False, None, True, None, None),
    ("a lane with no keys", 128, 128, 64, 2, 2, False, [100, 0], False, None, None),
    ("a negative scale", 128, 128, 64, 2, 2, True, [128, 50], False, -0.1, None),
    ("d 128, gqa, ragged, long enough for the hot loop", 300, 420, 128, 4, 2, True, [420, 299], False, None, None),
    ("d 64, 640 keys", 256, 640, 64, 2, 2, False, [640, 333], False, None, None),
    ("four splits", 128, 200, 64, 4, 4, False, [200, 70], False, None, 4),
]


@pytest.mark.parametrize("name,t,tk,d,h,hkv,causal,lens,key_mask,scale,splits", CASES, ids=[c[0] for c in CASES])
def test_f16_attention_matches_a_direct_softmax(device, name, t, tk, d, h, hkv, causal, lens, key_mask, scale, splits):
    q, k, v = case(t, tk, d, h, hkv)
    mask = None
    keys = KeyMask.none()
    if key_mask:
        b, j = np.meshgrid(np.arange(2), np.arange(tk), indexing="ij")
        mask = (b + j) % 5 != 2  # attention.rs:80-81
        keys = KeyMask.bool(torch.from_numpy(mask).to(device))
    elif lens is not None:
        keys = KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    got = svod_amd.attention(f16_tensor(q, device), f16_tensor(k, device), f16_tensor(v, device),
                             Attn(causal=causal, keys=keys, scale=scale, splits=splits))
    torch.cuda.synchronize()
    assert got.dtype == torch.float16
    assert "mfma_f32_32x32x16_f16" in svod_amd.chosen() or "combine_splits" in svod_amd.chosen(), svod_amd.chosen()
    got = to_np(got)
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=None if (lens is None or key_mask) else np.asarray(lens),
                           key_mask=mask, scale=scale)
    direct = oracle.attention_direct(p)
    with oracle.stream_dtype("f16"):
        program = oracle.attention_flash(p, bq=128, bkv=64, splits=splits or 1)
    assert np.isfinite(got).all()
    assert max_abs(got, direct) < 2e-2  # attention.rs:483
    assert max_abs(got, program) <= 2e-3
    if scale is None:
        # f16 carries three more mantissa bits than bf16: the 1e-3 bar holds against f64 itself.
        assert mean_rel(got, direct) <= 1e-3
        assert mean_rel(got, program) <= 5e-4


def test_f16_rows_no_key_reaches_are_zeros(device):
    q, k, v = case(128, 128, 64)
    lens = torch.tensor([0, 128], dtype=torch.int32, device=device)
    got = svod_amd.attention(f16_tensor(q, device), f16_tensor(k, device), f16_tensor(v, device), Attn(keys=KeyMask.lens(lens)))
    torch.cuda.synchronize()
    assert not f16_bits(got[0]).any()


def test_f16_packed_attention_is_the_split_call_bit_for_bit(device):
    b, t, h, hkv, d = 2, 130, 4, 2, 64
    x = f16_tensor(oracle.round_f16(Lcg(31).bf16((b, t, (h + 2 * hkv) * d))), device)
    q, k, v = (p.contiguous() for p in x.split([h * d, hkv * d, hkv * d], dim=-1))
    opts = Attn(causal=True)
    packed = svod_amd.attention_packed(x, h, hkv, opts)
    split = svod_amd.attention(q.view(b, t, h, d), k.view(b, t, hkv, d), v.view(b, t, hkv, d), opts)
    torch.cuda.synchronize()
    assert np.array_equal(f16_bits(packed), f16_bits(split))


@pytest.mark.parametrize("d,rope", [(64, False), (128, True), (32, None)], ids=["d 64 shared tables", "d 128 by token", "a split"])
def test_f16_heads_match_the_reference(device, d, rope):
    """heads.rs:112-161 with every operand f16."""
    batch, t, heads, kv_heads = 2, 37, 4, 2
    g = Lcg(11)
    slots, half = heads + 2 * kv_heads, d // 2
    r = oracle.round_f16
    qkv = r(g.bf16((batch, t, slots * d), mul=3.0))
    normed = rope is not None
    q_w = r(g.bf16((d,), mul=0.5, add=1.0)) if normed else None
    k_w = r(g.bf16((d,), mul=0.5, add=1.0)) if normed else None
    cos = sin = None
    if rope is not None:
        rows = batch * t if rope else t
        e = np.arange(rows * half)
        ang = (e // half).astype(np.float64) * 0.01 * (1.0 + (e % half).astype(np.float64))
        shape = (batch if rope else 1, t, 1, half)
        cos, sin = r(np.cos(ang).astype(np.float32)).reshape(shape), r(np.sin(ang).astype(np.float32)).reshape(shape)
    tt = lambda a: None if a is None else f16_tensor(a, device)
    opts = Qkv(heads=heads, kv_heads=kv_heads, head_dim=d, q_norm=tt(q_w), k_norm=tt(k_w), eps=1e-6,
               rope=None if cos is None else (tt(cos), tt(sin)))
    got = svod_amd.heads(tt(qkv), opts)
    torch.cuda.synchronize()
    p = oracle.HeadsProblem(qkv, heads, kv_heads, d, q_w, k_w, 1e-6, cos, sin)
    with oracle.stream_dtype("f16"):
        direct, program = oracle.heads_direct(p), oracle.heads_kernel(p)
    for i, what in enumerate("qkv"):
        gi = to_np(got[i])
        assert got[i].dtype == torch.float16 and np.isfinite(gi).all()
        assert max_abs(gi, direct[i]) <= 2e-2, what   # heads.rs:124
        assert max_abs(gi, program[i]) <= 2e-3, what  # one f16 step at |x| < 4 is 2^-9; the f32 work agrees far closer
    want_v = f16_tensor(qkv.reshape(batch, t, slots, d)[:, :, heads + kv_heads:, :], "cpu")
    assert np.array_equal(f16_bits(got[2]), f16_bits(want_v))
