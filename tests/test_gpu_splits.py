"""Key splits through the C ABI: the attention kernel's partial states merged by combine_splits
(tk/src/kernels/attention.rs:487-492, 609-612, 899-921, 948-1014; tk/src/ops/attention.rs:280-302).

Cases follow the reference's split tests in spirit (tk/src/test/unit/attention.rs:397-412,
tk/src/test/unit/ops.rs:585-628): several split counts, more splits than a row has blocks, a
lane with no keys, a negative scale's partial maxima, d 128.  The reference exercises splits
through its cache mode (tests/test_gpu_cache.py holds those cases); here the same split and merge
run on plain calls."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, assert_bf16_parity, bf16_tensor, bits, max_abs, to_np

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("key_tiles")]


def case(b, t, tk, h, hkv, d, seed=5):
    g = Lcg(seed)
    return g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))


def run(device, q, k, v, splits, causal=False, lens=None, mask=None, scale=None, workspace=None):
    keys = KeyMask.none()
    if lens is not None:
        keys = KeyMask.lens(torch.tensor(np.asarray(lens), dtype=torch.int32, device=device))
    if mask is not None:
        keys = KeyMask.bool(torch.from_numpy(np.ascontiguousarray(mask)).to(device))
    o = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                           Attn(causal=causal, keys=keys, scale=scale, splits=splits), workspace=workspace)
    torch.cuda.synchronize()
    return o


# (name, b, t, tk, h, hkv, d, splits, causal, lens, scale)
CASES = [
    ("one query, 1500 keys, four splits", 1, 1, 1500, 20, 20, 64, 4, False, None, None),  # ops.rs:585
    ("three queries, two splits", 2, 3, 200, 4, 4, 64, 2, False, [200, 70], None),       # ops.rs:587
    ("four splits, key lengths", 2, 128, 200, 4, 4, 64, 4, False, [200, 70], None),      # attention.rs:397
    ("d 128, two splits, five queries", 2, 5, 96, 2, 2, 128, 2, False, [64, 96], None),  # attention.rs:398
    ("more splits than blocks for a row", 2, 1, 64, 2, 2, 64, 4, False, [64, 40], None),  # attention.rs:399
    ("a lane with no keys, four splits", 2, 1, 200, 4, 4, 64, 4, False, [0, 70], None),  # attention.rs:411
    ("a negative scale's partial maxima", 2, 64, 200, 4, 4, 64, 4, True, [200, 70], -0.1),  # attention.rs:412
    ("causal, three splits, gqa", 2, 256, 256, 8, 2, 64, 3, True, [256, 130], None),
    ("causal d 128, two splits, ragged", 1, 200, 200, 4, 2, 128, 2, True, None, None),
    ("seven splits of seven blocks", 1, 128, 448, 2, 2, 64, 7, False, None, None),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,splits,causal,lens,scale", CASES, ids=[c[0] for c in CASES])
def test_split_attention_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, d, splits, causal, lens, scale):
    q, k, v = case(b, t, tk, h, hkv, d)
    got = to_np(run(device, q, k, v, splits, causal, lens, scale=scale))
    want_splits = min(splits, -(-tk // 64))
    if want_splits > 1:
        assert svod_amd.chosen().startswith('Kernel { op: "attention", family: "combine_splits"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, k, v, causal=causal, key_lens=None if lens is None else np.asarray(lens), scale=scale)
    direct = oracle.attention_direct(p)
    program = oracle.attention_flash(p, bq=128, bkv=64, splits=want_splits)
    assert np.isfinite(got).all()
    assert max_abs(got, direct) < 2e-2  # attention.rs:483
    assert max_abs(got, program) <= 1e-2
    if scale is None:
        assert_bf16_parity(name, got, direct, program)


def test_splits_change_only_the_merge(device):
    """A split call and an unsplit one see the same keys: they agree to the rounding of the
    merge (one exp2 and two multiplies per part), far inside one bf16 step of the values."""
    q, k, v = case(2, 256, 512, 4, 4, 64, seed=11)
    lens = [512, 300]
    whole = to_np(run(device, q, k, v, None, lens=lens))
    for splits in (2, 4, 8):
        part = to_np(run(device, q, k, v, splits, lens=lens))
        assert max_abs(part, whole) <= 2 ** -7, splits


def test_rows_no_key_reaches_are_zeros_in_every_split(device):
    """Every part of such a row holds l = 0 and o = 0: the merge divides by 1 (attention.rs:971-980)."""
    q, k, v = case(2, 130, 300, 4, 4, 64)
    got = run(device, q, k, v, 4, lens=[0, 300])
    assert not bits(got[0]).any()
    assert np.abs(to_np(got[1])).max() > 0


def test_one_split_or_none_is_the_unsplit_kernel(device):
    q, k, v = case(1, 64, 128, 2, 2, 64)
    a = run(device, q, k, v, None)
    assert svod_amd.chosen().startswith('Kernel { op: "attention", family: "flash_attention"')
    b = run(device, q, k, v, 1)
    assert svod_amd.chosen().startswith('Kernel { op: "attention", family: "flash_attention"')
    assert np.array_equal(bits(a), bits(b))


def test_a_split_call_without_room_keeps_the_graph(device):
    """The reference op allocates the partial tensors; here they are the caller's.  A workspace
    that cannot hold them means no kernel config applies."""
    q, k, v = case(1, 64, 256, 2, 2, 64)
    small = torch.empty(1024, dtype=torch.uint8, device=device)
    with pytest.raises(svod_amd.GraphFallback) as e:
        run(device, q, k, v, 2, workspace=small)
    assert e.value.why == svod_amd.Fallback.Config


def test_full_size_split_equals_unsplit(device):
    """The long-context shape (B2 H16 d64 S8192, lens {8192, 5000}) with four splits against the
    unsplit kernel: the same keys, merged."""
    from svod_amd import workloads as W
    w = W.config5(device=device)
    keys = KeyMask.lens(w.key_lens)
    whole = svod_amd.attention(w.q, w.k, w.v, Attn(keys=keys, scale=w.scale))
    part = svod_amd.attention(w.q, w.k, w.v, Attn(keys=keys, scale=w.scale, splits=4))
    torch.cuda.synchronize()
    diff = (whole.float() - part.float()).abs().max().item()
    assert diff <= 2 ** -8, diff


# ---- attention_packed (tk/src/ops/attention.rs:104-122)
def packed_case(b, t, h, hkv, d, seed=31):
    return Lcg(seed).bf16((b, t, (h + 2 * hkv) * d))


@pytest.mark.parametrize("b,t,h,hkv,d,causal,lens,splits", [
    (2, 100, 4, 4, 64, False, [100, 61], None),
    (2, 200, 8, 2, 64, True, None, None),
    (1, 130, 4, 2, 128, True, [99], None),
    (2, 256, 4, 4, 64, False, [256, 70], 2),
], ids=["lens", "causal gqa", "d 128 causal gqa ragged", "two splits"])
def test_packed_attention_is_the_split_call_bit_for_bit(device, b, t, h, hkv, d, causal, lens, splits):
    """ops.rs:519-521: the packed kernel and the kernel over the three split tensors agree bit for bit;
    and the packed call sits on the direct softmax like any other."""
    x = packed_case(b, t, h, hkv, d)
    xt = bf16_tensor(x, device)
    q, k, v = (p.contiguous() for p in xt.split([h * d, hkv * d, hkv * d], dim=-1))
    q, k, v = q.view(b, t, h, d), k.view(b, t, hkv, d), v.view(b, t, hkv, d)
    keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    opts = Attn(causal=causal, keys=keys, splits=splits)
    packed = svod_amd.attention_packed(xt, h, hkv, opts)
    split = svod_amd.attention(q, k, v, opts)
    torch.cuda.synchronize()
    assert np.array_equal(bits(packed), bits(split))
    p = oracle.AttnProblem(to_np(q), to_np(k), to_np(v), causal=causal, key_lens=None if lens is None else np.asarray(lens))
    assert max_abs(to_np(packed), oracle.attention_direct(p)) < 2e-2


def test_a_decoder_step_is_split_unasked_when_the_workspace_is_lent(device):
    """One query row against 8192 keys: with no count named the library splits the keys (and merges),
    given the workspace it asks for; without one it keeps them whole.  Both agree with the direct softmax."""
    b, t, tk, h, hkv, d = 1, 1, 8192, 8, 2, 64
    g = Lcg(17)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    dq, dk, dv = (bf16_tensor(x, device) for x in (q, k, v))
    want = oracle.attention_direct(oracle.AttnProblem(q, k, v))
    split = svod_amd.attention(dq, dk, dv)  # the wrapper lends what svodk_attention_workspace asks for
    assert "combine_splits" in svod_amd.chosen()
    whole = svod_amd.attention(dq, dk, dv, workspace=torch.empty(16, dtype=torch.uint8, device=device))
    assert "combine_splits" not in svod_amd.chosen() and "flash_attention" in svod_amd.chosen()
    one = svod_amd.attention(dq, dk, dv, Attn(splits=1))
    assert "combine_splits" not in svod_amd.chosen()
    torch.cuda.synchronize()
    assert np.array_equal(bits(whole), bits(one))
    for got in (split, whole):
        assert max_abs(to_np(got), want) < 2e-2
