"""svodk_attention_noalloc through the C ABI: the entry point for callers that cannot allocate keeps
the partial states of a split call in the library's static device array.  Its output is held bit for
bit to svodk_attention's with a lent workspace (the same kernels on the same operands), on two calls
in a row, the second with a smaller input, so what the first call left in the array cannot show."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, Cache, KeyMask, OpError
from util import Lcg, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu


def operands(device, b, t, tk, h, hkv, d, seed):
    g = Lcg(seed)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    return (q, k, v), tuple(bf16_tensor(x, device) for x in (q, k, v))


def both(device, dev_ops, opts):
    q, k, v = dev_ops
    want = svod_amd.attention(q, k, v, opts)  # lends a workspace of its own
    chosen_want = svod_amd.chosen()
    out = torch.full_like(q, float("nan"))
    # Neither torch's allocator nor the device itself gives anything out under the call: the second
    # figure is the device's free bytes (a hipMalloc inside the library would lower it).
    torch.cuda.synchronize()
    before, free_before = torch.cuda.memory_allocated(device), torch.cuda.mem_get_info(device)[0]
    got = svod_amd.attention_noalloc(q, k, v, opts, out)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(device) == before
    assert torch.cuda.mem_get_info(device)[0] == free_before
    assert svod_amd.chosen() == chosen_want
    torch.cuda.synchronize()
    return got, want


def test_two_calls_in_a_row_match_the_lent_workspace(device):
    # A decoder step with four named splits, then a smaller one with three over fewer rows: the
    # second call's partial states cover a part of what the first left behind.
    for (b, t, tk, h, hkv, d, splits, lens, seed) in [(4, 3, 1500, 8, 8, 64, 4, [1500, 900, 64, 0], 5),
                                                      (2, 1, 700, 4, 2, 128, 3, [700, 130], 9)]:
        host, dev_ops = operands(device, b, t, tk, h, hkv, d, seed)
        keys = KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
        got, want = both(device, dev_ops, Attn(keys=keys, splits=splits))
        assert svod_amd.chosen().startswith('Kernel { op: "attention", family: "combine_splits"'), svod_amd.chosen()
        assert np.array_equal(bits(got), bits(want))
        p = oracle.AttnProblem(*host, key_lens=np.asarray(lens))
        assert max_abs(to_np(got), oracle.attention_direct(p)) < 2e-2  # tk/src/test/unit/attention.rs:483


def test_the_library_chooses_splits_as_with_a_workspace(device):
    # splits = None: the rule's own count, taken as if a workspace had been lent.
    host, dev_ops = operands(device, 2, 1, 4096, 8, 2, 128, seed=13)
    got, want = both(device, dev_ops, Attn())
    assert svod_amd.chosen().startswith('Kernel { op: "attention", family: "combine_splits"'), svod_amd.chosen()
    assert np.array_equal(bits(got), bits(want))
    # An unsplit call needs no scratch and runs as svodk_attention does.
    host, dev_ops = operands(device, 2, 200, 200, 4, 2, 64, seed=17)
    got, want = both(device, dev_ops, Attn(causal=True))
    assert np.array_equal(bits(got), bits(want))


def test_a_call_past_the_scratch_is_refused(device):
    cap = svod_amd.noalloc_scratch_bytes()
    assert cap == 8 << 20
    b, t, h, d, splits = 4, 128, 16, 128, 4
    assert splits * b * t * h * (d + 2) * 4 > cap
    _, (q, k, v) = operands(device, b, t, 512, h, h, d, seed=3)
    out = torch.full_like(q, float("nan"))
    with pytest.raises(OpError) as e:
        svod_amd.attention_noalloc(q, k, v, Attn(splits=splits), out)
    assert e.value.kind == "Argument" and "static scratch holds" in str(e.value)
    torch.cuda.synchronize()
    assert torch.isnan(out).all()  # nothing was launched


def test_splits_of_the_rules_own_shrink_to_the_scratch(device):
    # splits = None on a prefill whose rule asks for 2 splits of 17 MB each: past the 8 MiB array the
    # count drops to one, as svodk_attention drops it without a workspace, and the call runs unsplit.
    b, t, tk, h, d = 1, 2048, 2048, 16, 128
    assert 2 * b * t * h * (d + 2) * 4 > svod_amd.noalloc_scratch_bytes()
    _, (q, k, v) = operands(device, b, t, tk, h, h, d, seed=21)
    out = torch.full_like(q, float("nan"))
    got = svod_amd.attention_noalloc(q, k, v, Attn(), out)
    assert svod_amd.chosen().startswith('Kernel { op: "attention", family: "flash_attention"'), svod_amd.chosen()
    want = svod_amd.attention(q, k, v, Attn(splits=1))
    torch.cuda.synchronize()
    assert np.array_equal(bits(got), bits(want))


def test_a_captured_split_call_replays(device):
    # The callers the entry point is for: a split call captured in a HIP graph (after one eager call on
    # the device, which looks the array's address up) and replayed with eager work between the replays.
    host, dev_ops = operands(device, 2, 1, 2048, 8, 2, 128, seed=29)
    q, k, v = dev_ops
    opts = Attn(splits=4)
    eager = svod_amd.attention_noalloc(q, k, v, opts, torch.full_like(q, float("nan")))
    torch.cuda.synchronize()
    out = torch.full_like(q, float("nan"))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        svod_amd.attention_noalloc(q, k, v, opts, out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        svod_amd.attention_noalloc(q, k, v, opts, out)
    for _ in range(3):
        out.fill_(float("nan"))
        # eager work on the same array between the replays: a smaller split call
        svod_amd.attention_noalloc(q[:1], k[:1], v[:1], Attn(splits=2), torch.empty_like(q[:1]))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits(out), bits(eager))
