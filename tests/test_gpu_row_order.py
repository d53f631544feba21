"""The batch row order of a launch (svodk_attn.row_order, svodk_order_rows): which row a workgroup takes
is free, so any permutation gives the same bits; the one svodk_order_rows computes is the rows in
descending order of their key lengths, ties by row."""
import numpy as np
import pytest
import torch

import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, bf16_tensor, bits

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,dtype", [(1, torch.int32), (5, torch.int64), (64, torch.int32), (300, torch.int32),
                                     (1500, torch.int64)])
def test_order_rows_is_a_stable_descending_sort(device, n, dtype):
    rng = np.random.default_rng(n)
    lens = rng.integers(0, 40, size=n)  # many ties
    got = svod_amd.order_rows(torch.from_numpy(lens).to(dtype).to(device)).cpu().numpy()
    want = np.argsort(-lens, kind="stable")
    assert np.array_equal(got, want)
    assert svod_amd.chosen().startswith('Kernel { op: "order_rows"')


@pytest.mark.parametrize("dtype", [torch.bool, torch.int32])
def test_order_rows_of_a_key_mask_counts_up_to_the_last_visible_key(device, dtype):
    rng = np.random.default_rng(4)
    n, tk = 37, 300
    mask = rng.random((n, tk)) < 0.02
    mask[5] = False                      # a row of nothing sorts last
    mask[9, tk - 1] = True               # a full-length row sorts first
    reach = np.where(mask.any(1), tk - np.argmax(mask[:, ::-1], axis=1), 0)
    got = svod_amd.order_rows(torch.from_numpy(mask).to(dtype).to(device)).cpu().numpy()
    assert np.array_equal(got, np.argsort(-reach, kind="stable"))
    assert got[0] == 9 and got[-1] == 5


# (b, t, tk, h, hkv, d, causal, splits)
CASES = [(12, 300, 300, 4, 2, 64, False, None), (7, 200, 260, 4, 4, 128, True, None), (5, 130, 512, 2, 2, 64, False, 2)]


@pytest.mark.parametrize("b,t,tk,h,hkv,d,causal,splits", CASES)
def test_any_row_order_gives_the_same_bits(device, b, t, tk, h, hkv, d, causal, splits):
    g = Lcg(21)
    q, k, v = (bf16_tensor(x, device) for x in (g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))))
    lens = torch.tensor([(37 * i) % (tk + 1) for i in range(b)], dtype=torch.int32, device=device)
    opts = dict(causal=causal, keys=KeyMask.lens(lens), splits=splits)
    plain = bits(svod_amd.attention(q, k, v, Attn(**opts)))
    longest_first = svod_amd.order_rows(lens)
    assert np.array_equal(bits(svod_amd.attention(q, k, v, Attn(row_order=longest_first, **opts))), plain)
    backwards = torch.arange(b - 1, -1, -1, dtype=torch.int32, device=device)
    assert np.array_equal(bits(svod_amd.attention(q, k, v, Attn(row_order=backwards, **opts))), plain)


def test_a_row_order_is_validated(device):
    g = Lcg(2)
    q, k = bf16_tensor(g.bf16((3, 64, 2, 64)), device), bf16_tensor(g.bf16((3, 64, 2, 64)), device)
    with pytest.raises(svod_amd.OpError) as e:
        svod_amd.attention(q, k, k, Attn(row_order=torch.zeros(4, dtype=torch.int32, device=device)))
    assert e.value.kind == "Shape" and "row order" in str(e.value)
    with pytest.raises(svod_amd.OpError) as e:
        svod_amd.attention(q, k, k, Attn(row_order=torch.zeros(3, dtype=torch.int64, device=device)))
    assert e.value.kind == "Dtype"
    # Entries out of range are clamped, never followed out of the tensors.
    wild = torch.tensor([-5, 1, 99], dtype=torch.int32, device=device)
    out = svod_amd.attention(q, k, k, Attn(row_order=wild))
    torch.cuda.synchronize()
    assert out.shape == q.shape


def test_an_order_that_is_no_permutation_leaves_the_rows_it_skips_unwritten(device):
    """The order's contents are device data no host check reads: the rows an order names are computed as ever, the
    rows it leaves out stay as the caller's buffer had them (here the harness's NaN fill), and nothing else happens."""
    g = Lcg(6)
    q, k, v = (bf16_tensor(x, device) for x in (g.bf16((4, 70, 2, 64)), g.bf16((4, 90, 2, 64)), g.bf16((4, 90, 2, 64))))
    whole = svod_amd.attention(q, k, v, Attn())
    twice = torch.tensor([2, 0, 2, 0], dtype=torch.int32, device=device)  # rows 1 and 3 are never named
    got = svod_amd.attention(q, k, v, Attn(row_order=twice))
    torch.cuda.synchronize()
    assert np.array_equal(bits(got[[0, 2]]), bits(whole[[0, 2]]))
    assert torch.isnan(got[[1, 3]].float()).all()


def misaligned_like(t):
    """The same values at an address one element past a 16-byte boundary (dense, but off the kernels' alignment)."""
    flat = torch.empty(t.numel() + 8, dtype=t.dtype, device=t.device)
    view = flat[1:1 + t.numel()].view(t.shape)
    view.copy_(t)
    return view


def test_addresses_off_the_kernels_alignment_are_refused(device):
    g = Lcg(8)
    q, k = bf16_tensor(g.bf16((2, 64, 2, 64)), device), bf16_tensor(g.bf16((2, 64, 2, 64)), device)
    for args in ((misaligned_like(q), k, k), (q, misaligned_like(k), k), (q, k, misaligned_like(k))):
        with pytest.raises(svod_amd.OpError) as e:
            svod_amd.attention(*args, Attn())
        assert e.value.kind == "Argument" and "aligned" in str(e.value)
    with pytest.raises(svod_amd.OpError) as e:
        svod_amd.attention(q, k, k, Attn(), out=misaligned_like(q))
    assert e.value.kind == "Argument" and "out is not 16-byte aligned" in str(e.value)
    x = bf16_tensor(g.bf16((2, 8, 512)), device)
    w = bf16_tensor(g.bf16((512,)), device)
    with pytest.raises(svod_amd.OpError) as e:
        svod_amd.rms_norm(misaligned_like(x), w)
    assert e.value.kind == "Argument" and "aligned" in str(e.value)
    with pytest.raises(svod_amd.OpError) as e:
        svod_amd.heads(misaligned_like(x), svod_amd.Qkv(4, 2, 64))
    assert e.value.kind == "Argument" and "aligned" in str(e.value)
