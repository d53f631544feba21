"""An additive bias (Attn::bias, tk/src/ops/attention.rs:82-85; biased() and the scaled-maximum step,
tk/src/kernels/attention.rs:355-370, 401-405, 566-571) through the C ABI against the oracle.  The first
cases are the reference's own (tk/src/test/unit/ops.rs:447-451, 456; tk/src/test/unit/attention.rs:296-300)
at the head sizes this library has kernels for, with its bias fixture's spread (2 x the generator)."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, assert_bf16_parity, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu


def case(b, t, tk, h, hkv, d, rows, seed=5):
    g = Lcg(seed)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    return q, k, v, g.bf16((rows, h, t, tk), mul=2.0)


# (name, b, t, tk, h, hkv, d, bias rows, masks, lens, splits)
CASES = [
    ("bias per batch", 2, 100, 100, 4, 4, 64, 2, {}, None, None),                                  # ops.rs:447
    ("d128 gqa causal shared bias", 2, 130, 130, 4, 2, 128, 1, dict(causal=True), None, None),     # ops.rs:448
    ("bias with key lens", 2, 99, 99, 4, 4, 64, 2, {}, [99, 50], None),                            # ops.rs:449
    ("biased cross attention", 2, 37, 150, 4, 4, 64, 2, {}, None, None),                           # ops.rs:450
    ("bias over packed segments", 2, 200, 200, 4, 2, 64, 1, dict(causal=True, seg=30), None, None),  # ops.rs:451
    ("every mask and a shared bias", 2, 128, 128, 2, 2, 64, 1,
     dict(causal=True, window=(50, 0), chunk=(32, 3, 0), seg=40), [128, 100], None),               # attention.rs:300
    ("keys off the 8-byte grid", 1, 70, 131, 2, 2, 64, 1, {}, None, None),
    ("long rows, several tiles", 1, 600, 700, 2, 1, 64, 1, {}, [650], None),
    ("d128 long causal", 1, 500, 500, 2, 2, 128, 1, dict(causal=True), None, None),
    ("two splits", 1, 300, 512, 2, 2, 64, 1, {}, None, 2),
    ("three splits under a window", 2, 256, 640, 2, 2, 64, 2, dict(window=(200, 100)), None, 3),
]


def run(device, b, t, tk, h, hkv, d, rows, masks, lens, splits, f16=False):
    q, k, v, bias = case(b, t, tk, h, hkv, d, rows)
    masks = dict(masks)
    seg = np.tile(np.arange(t) - np.arange(t) % masks.pop("seg"), (b, 1)) if "seg" in masks else None
    keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    seg_t = None if seg is None else torch.from_numpy(seg).to(torch.int32).to(device)
    if f16:
        q, k, v, bias = (oracle.round_f16(x) for x in (q, k, v, bias))
        up = lambda x: torch.from_numpy(x).to(torch.float16).to(device)
    else:
        up = lambda x: bf16_tensor(x, device)
    got = svod_amd.attention(up(q), up(k), up(v), Attn(keys=keys, seg_start=seg_t, bias=up(bias), splits=splits, **masks))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, k, v, key_lens=None if lens is None else np.asarray(lens), seg_start=seg, bias=bias, **masks)
    return got, p


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,rows,masks,lens,splits", CASES, ids=[c[0] for c in CASES])
def test_biased_attention_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, d, rows, masks, lens, splits):
    got, p = run(device, b, t, tk, h, hkv, d, rows, masks, lens, splits)
    direct = oracle.attention_direct(p)
    program = oracle.attention_flash(p, bq=128, bkv=64, splits=splits or 1)
    assert_bf16_parity(name, to_np(got), direct, program)


def test_f16_biased_causal(device):
    """tk/src/test/unit/ops.rs:456."""
    got, p = run(device, 1, 70, 70, 2, 2, 64, 1, dict(causal=True), None, None, f16=True)
    with oracle.stream_dtype("f16"):
        program = oracle.attention_flash(p, bq=128, bkv=64)
    direct = oracle.attention_direct(p)
    got = got.detach().cpu().to(torch.float32).numpy()
    assert max_abs(got, direct) < 2e-2
    assert max_abs(got, program) < 2e-2


def test_bias_closed_forms(device):
    b, t, tk, h, d = 2, 150, 200, 2, 64
    q, k, v, bias = case(b, t, tk, h, h, d, 2)
    dq, dk, dv = (bf16_tensor(x, device) for x in (q, k, v))
    plain = to_np(svod_amd.attention(dq, dk, dv))
    # The same number added to every score of a row leaves its softmax unchanged (up to the
    # rounding of the sum s*scale*log2e + c*log2e).
    flat = np.broadcast_to(np.linspace(-3, 3, t, dtype=np.float32)[None, None, :, None], bias.shape)
    shifted = to_np(svod_amd.attention(dq, dk, dv, Attn(bias=bf16_tensor(np.ascontiguousarray(flat), device))))
    assert max_abs(shifted, plain) < 2e-2
    # A bias of -inf on a key is a key mask, and a row of nothing but -inf is a row of zeros.
    hide = np.add.outer(np.arange(b), np.arange(tk)) % 5 == 2
    walls = np.where(hide[:, None, None, :], -np.inf, 0.0).astype(np.float32) * np.ones_like(bias)
    walls[1, :, 7, :] = -np.inf
    got = to_np(svod_amd.attention(dq, dk, dv, Attn(bias=bf16_tensor(walls, device))))
    masked = to_np(svod_amd.attention(dq, dk, dv, Attn(keys=KeyMask.bool(torch.from_numpy(~hide).to(device)))))
    keep = np.ones((b, t), dtype=bool)
    keep[1, 7] = False
    assert max_abs(got[keep], masked[keep]) < 2e-2
    assert not got[1, 7].any()
    # Zero queries: the bias alone sets the weights, one-hot values read them out.
    one_hot = np.zeros((b, tk, h, d), dtype=np.float32)
    for c in range(d):
        one_hot[:, 100 + c, :, c] = 1.0
    got = to_np(svod_amd.attention(bf16_tensor(np.zeros_like(q), device), dk, bf16_tensor(one_hot, device),
                                   Attn(bias=bf16_tensor(bias, device))))
    w = np.exp(bias.astype(np.float64))
    w /= w.sum(-1, keepdims=True)
    assert max_abs(got, w[:, :, :, 100:100 + d].transpose(0, 2, 1, 3)) < 1e-3


def test_a_shared_bias_is_the_per_batch_bias_repeated(device):
    b, t, tk, h, d = 3, 90, 130, 2, 64
    q, k, v, bias = case(b, t, tk, h, h, d, 1)
    dq, dk, dv = (bf16_tensor(x, device) for x in (q, k, v))
    shared = svod_amd.attention(dq, dk, dv, Attn(bias=bf16_tensor(bias, device)))
    repeated = svod_amd.attention(dq, dk, dv, Attn(bias=bf16_tensor(np.repeat(bias, b, axis=0), device)))
    assert np.array_equal(bits(shared), bits(repeated))


def test_a_bias_off_the_stream_dtype_keeps_the_graph(device):
    """tk/src/ops/attention.rs:84-85 and shape.rs:92-99."""
    q, k, v, bias = case(1, 64, 64, 2, 2, 64, 1)
    with pytest.raises(svod_amd.GraphFallback) as e:
        svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                           Attn(bias=torch.from_numpy(bias).to(torch.float16).to(device)))
    assert e.value.why == svod_amd.Fallback.Dtype


@pytest.mark.parametrize("per_key,causal", [(0.1, False), (1.0, False), (0.1, True)],
                         ids=["a slow climb", "a steep climb", "a slow causal climb"])
def test_climbing_scores_rescale_the_accumulator(device, per_key, causal):
    """attention.rs:457-472: a bias ramp along the keys (per_key * j, rounded to bf16).  Slowly, a row keeps
    its stale maximum for several blocks and then adopts a new one; steeply, it adopts one every block.
    Either way the accumulator is rescaled while it holds earlier blocks' work.  384 keys here (the
    reference's 128 are two of this kernel's key blocks)."""
    b, t, tk, h, d = 2, 128, 384, 2, 64
    q, k, v, _ = case(b, t, tk, h, h, d, b)
    ramp = oracle.round_bf16((per_key * np.arange(tk)).astype(np.float32))
    bias = np.ascontiguousarray(np.broadcast_to(ramp, (b, h, t, tk))).astype(np.float32)
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                             Attn(causal=causal, bias=bf16_tensor(bias, device)))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, k, v, causal=causal, bias=bias)
    assert_bf16_parity("climbing bias", to_np(got), oracle.attention_direct(p), oracle.attention_flash(p, bq=128, bkv=64))
