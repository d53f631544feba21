"""The streaming form of the attention kernel (workgroups that walk query tiles one after another,
the next tile's first key blocks and Q rows fetched under the current tile's steps, tiles handed
out by a shared counter) against the one-tile form: a tile's arithmetic is the same steps in the
same order, so the two agree bit for bit whichever workgroup takes which tile.  The knob forces
streaming with few workgroups, so that walks are long and cross heads, batch rows, one-block
tiles, odd and even block counts and idle causal waves."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, KeyMask
from util import Lcg, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def automatic_again():
    yield
    svod_amd.tune_streaming(0)


def case(b, t, tk, h, hkv, d=64, seed=13):
    g = Lcg(seed)
    return g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))


# (name, b, t, tk, h, hkv, causal, lens)
CASES = [
    ("ragged lengths, one to eight blocks", 12, 512, 512, 4, 4, False, [64, 65, 512, 1, 128, 300, 0, 449, 191, 192, 193, 7]),
    ("no mask, odd block count", 3, 300, 320, 2, 2, False, None),
    ("causal gqa", 4, 384, 384, 8, 2, True, None),
    ("causal with lengths", 5, 256, 256, 4, 4, True, [256, 50, 0, 129, 64]),
    ("one query row, many keys", 9, 1, 700, 2, 2, False, [700, 1, 64, 128, 129, 500, 0, 699, 65]),
    ("cross attention, more heads than units per XCD", 2, 130, 90, 16, 8, False, [90, 33]),
]


@pytest.mark.parametrize("slots", [1, 2, 5, 96], ids=["1 workgroup an XCD", "2", "5", "more workgroups than tiles"])
@pytest.mark.parametrize("name,b,t,tk,h,hkv,causal,lens", CASES, ids=[c[0] for c in CASES])
def test_streaming_is_the_one_tile_kernel_bit_for_bit(device, name, b, t, tk, h, hkv, causal, lens, slots):
    q, k, v = (bf16_tensor(x, device) for x in case(b, t, tk, h, hkv))
    keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    opts = Attn(causal=causal, keys=keys)
    svod_amd.tune_streaming(-1)
    plain = svod_amd.attention(q, k, v, opts)
    svod_amd.tune_streaming(slots)
    streamed = svod_amd.attention(q, k, v, opts)
    torch.cuda.synchronize()
    assert np.array_equal(bits(streamed), bits(plain))


def test_streaming_matches_a_direct_softmax(device):
    b, t, tk, h, hkv = 6, 200, 260, 4, 2
    q, k, v = case(b, t, tk, h, hkv)
    lens = [260, 1, 64, 200, 0, 131]
    svod_amd.tune_streaming(3)
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device),
                             Attn(keys=KeyMask.lens(torch.tensor(lens, dtype=torch.int64, device=device))))
    torch.cuda.synchronize()
    p = oracle.AttnProblem(q, k, v, key_lens=np.asarray(lens))
    assert max_abs(to_np(got), oracle.attention_direct(p)) < 2e-2
    assert not bits(got[4]).any()  # the batch row with no keys


def test_streaming_f16_and_packed(device):
    b, t, h, hkv, d = 5, 190, 4, 2, 64
    x = torch.from_numpy(oracle.round_f16(Lcg(3).bf16((b, t, (h + 2 * hkv) * d)))).to(torch.float16).to(device)
    opts = Attn(causal=True, keys=KeyMask.lens(torch.tensor([190, 64, 1, 0, 100], dtype=torch.int32, device=device)))
    svod_amd.tune_streaming(-1)
    plain = svod_amd.attention_packed(x, h, hkv, opts)
    svod_amd.tune_streaming(2)
    streamed = svod_amd.attention_packed(x, h, hkv, opts)
    torch.cuda.synchronize()
    a, c = (y.detach().cpu().view(torch.int16).numpy() for y in (plain, streamed))
    assert np.array_equal(a, c)


def test_counters_are_left_at_zero_for_the_launch_that_meets_them_next(device):
    """Launches take the sets of shared counters in turn (256 of them): well past one turn of the
    sets, every launch still hands out every tile once."""
    q, k, v = (bf16_tensor(x, device) for x in case(3, 260, 200, 4, 2, seed=29))
    opts = Attn(keys=KeyMask.lens(torch.tensor([200, 77, 129], dtype=torch.int32, device=device)))
    svod_amd.tune_streaming(-1)
    plain = bits(svod_amd.attention(q, k, v, opts))
    svod_amd.tune_streaming(2)
    out = torch.empty_like(q)
    for launch in range(600):
        if launch % 100 == 99:
            out.zero_()
        svod_amd.attention(q, k, v, opts, out=out)
        if launch % 100 == 99:
            torch.cuda.synchronize()
            assert np.array_equal(bits(out), plain), launch


def test_two_streams_at_once_do_not_share_counters(device):
    q1, k1, v1 = (bf16_tensor(x, device) for x in case(4, 512, 512, 8, 8, seed=5))
    q2, k2, v2 = (bf16_tensor(x, device) for x in case(2, 700, 700, 4, 2, seed=6))
    causal = Attn(causal=True)
    svod_amd.tune_streaming(-1)
    want1, want2 = bits(svod_amd.attention(q1, k1, v1)), bits(svod_amd.attention(q2, k2, v2, causal))
    svod_amd.tune_streaming(3)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    o1, o2 = torch.empty_like(q1), torch.empty_like(q2)
    torch.cuda.synchronize()
    for _ in range(20):
        with torch.cuda.stream(s1):
            svod_amd.attention(q1, k1, v1, out=o1)
        with torch.cuda.stream(s2):
            svod_amd.attention(q2, k2, v2, causal, out=o2)
    torch.cuda.synchronize()
    assert np.array_equal(bits(o1), want1)
    assert np.array_equal(bits(o2), want2)


def test_streaming_follows_a_row_order(device):
    b, t, tk, h, hkv = 9, 300, 300, 4, 2
    q, k, v = (bf16_tensor(x, device) for x in case(b, t, tk, h, hkv, seed=41))
    lens = torch.tensor([300, 7, 64, 129, 0, 255, 300, 65, 1], dtype=torch.int32, device=device)
    order = svod_amd.order_rows(lens)
    svod_amd.tune_streaming(-1)
    plain = bits(svod_amd.attention(q, k, v, Attn(keys=KeyMask.lens(lens))))
    svod_amd.tune_streaming(3)
    streamed = svod_amd.attention(q, k, v, Attn(keys=KeyMask.lens(lens), row_order=order))
    torch.cuda.synchronize()
    assert np.array_equal(bits(streamed), plain)


def test_a_captured_call_takes_no_counter_set(device):
    """Under stream capture the knob is not followed: a graph's replays would share the one set of
    tile counters the capture took.  The captured call runs a workgroup per tile, so it takes no
    set, and every replay gives the eager result."""
    lib = svod_amd.load_library()
    sets = 256
    q, k, v = (bf16_tensor(x, device) for x in case(4, 384, 384, 8, 2))
    opts = Attn(causal=True)
    svod_amd.tune_streaming(-1)
    plain = svod_amd.attention(q, k, v, opts)
    svod_amd.tune_streaming(3)
    before = lib.svodk_streaming_next_set()
    streamed = svod_amd.attention(q, k, v, opts)  # eager: streams, takes the next set
    torch.cuda.synchronize()
    assert (lib.svodk_streaming_next_set() - before) % sets == 2
    out = torch.empty_like(plain)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        svod_amd.attention(q, k, v, opts, out=out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    before = lib.svodk_streaming_next_set()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        svod_amd.attention(q, k, v, opts, out=out)
    assert (lib.svodk_streaming_next_set() - before) % sets == 1  # only this probe took one
    for _ in range(3):
        out.fill_(3.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert np.array_equal(bits(out), bits(plain))
    assert np.array_equal(bits(streamed), bits(plain))
