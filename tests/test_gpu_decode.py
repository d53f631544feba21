"""The decoder step's kernel: a call without causal or per-row masks or a bias whose KV heads each serve at most
four query rows (heads / kv_heads * T) streams K and V through registers (svod_amd/csrc/decode_kernel.hip) instead
of running key tiles.  Its results are the op's (tk/src/kernels/attention.rs:466-924) to the same bar as the tile
kernel's: against a float64 softmax of the same operands, and against the tile kernel itself on the same call."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, Cache, KeyMask
from util import Lcg, bf16_tensor, max_abs, mean_rel, to_np

STREAMED = "keys streamed through registers"


@pytest.fixture(autouse=True)
def up_to_four_rows():
    """Unasked the library sends one and two rows that way; the kernel is built for up to four."""
    svod_amd.tune_decode(4)
    yield
    svod_amd.tune_decode(svod_amd.DECODE_ROWS_DEFAULT)


pytestmark = pytest.mark.gpu


def both_paths(call):
    """The call on the decoder step's kernel and on key tiles."""
    got = call()
    torch.cuda.synchronize()
    split = "combine_splits" in svod_amd.chosen()  # the last kernel of a split call is the merge of its splits
    assert split or STREAMED in svod_amd.chosen(), svod_amd.chosen()
    svod_amd.tune_decode(0)
    try:
        tiles = call()
        torch.cuda.synchronize()
        assert STREAMED not in svod_amd.chosen(), svod_amd.chosen()
    finally:
        svod_amd.tune_decode(4)  # this module's setting (up_to_four_rows)
    return got, tiles


def check(name, got, tiles, want):
    g, t = to_np(got), to_np(tiles)
    assert np.isfinite(g).all(), name
    assert max_abs(g, want) < 2e-2, name
    assert mean_rel(g, want) < 2e-3, name
    assert max_abs(g, t) < 2e-2, name


# (name, b, t, tk, h, hkv, d, splits, lens)
SHAPES = [
    ("one row, d 64, 1500 keys", 3, 1, 1500, 5, 5, 64, None, None),
    ("one row, lengths incl. 0, 1, a block's edge", 6, 1, 300, 4, 4, 64, None, [300, 0, 1, 64, 65, 129]),
    ("one row, four splits named", 2, 1, 1000, 4, 4, 64, 4, [1000, 517]),
    ("more splits than blocks", 2, 1, 100, 4, 4, 64, 7, [100, 3]),
    ("group of four", 2, 1, 700, 8, 2, 64, None, [700, 33]),
    ("group of two, two tokens", 2, 2, 257, 4, 2, 64, None, None),
    ("three tokens, one head a KV head", 2, 3, 190, 3, 3, 64, 2, [190, 64]),
    ("group of three", 1, 1, 450, 6, 2, 64, None, None),
    ("d 32", 2, 1, 333, 4, 2, 32, None, [333, 17]),
    ("d 48", 2, 2, 333, 4, 2, 48, 3, [333, 200]),
    ("d 128, group of four", 2, 1, 900, 8, 2, 128, None, [900, 450]),
    ("d 128, split", 2, 1, 2100, 4, 4, 128, 5, None),
    ("d 256", 2, 1, 400, 4, 2, 256, None, [400, 5]),
    ("d 256, four rows, split", 1, 2, 500, 4, 2, 256, 2, None),
    ("a single key", 2, 1, 1, 4, 4, 64, None, None),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,splits,lens", SHAPES, ids=[c[0] for c in SHAPES])
def test_a_decoder_step_matches_a_direct_softmax(device, name, b, t, tk, h, hkv, d, splits, lens):
    g = Lcg(77)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    dev = lambda x: bf16_tensor(x, device)
    got, tiles = both_paths(lambda: svod_amd.attention(dev(q), dev(k), dev(v), Attn(keys=keys, splits=splits)))
    want = oracle.attention_direct(oracle.AttnProblem(q, k, v, key_lens=None if lens is None else np.asarray(lens)))
    check(name, got, tiles, want)


@pytest.mark.parametrize("kind", ["bool", "int"])
@pytest.mark.parametrize("d,splits", [(64, None), (128, 3)])
def test_key_masks_hide_keys_anywhere(device, kind, d, splits):
    b, t, tk, h, hkv = 4, 1, 700, 4, 2
    g = Lcg(5)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    rng = np.random.default_rng(3)
    mask = rng.random((b, tk)) < 0.6
    mask[1] = False          # a row that sees nothing: zeros
    mask[2, :] = True
    mask[3, 100:] = False    # a padding mask
    dev = lambda x: bf16_tensor(x, device)
    m = torch.from_numpy(mask).to(device) if kind == "bool" else torch.from_numpy(mask.astype(np.int32)).to(device)
    keys = KeyMask.bool(m)
    got, tiles = both_paths(lambda: svod_amd.attention(dev(q), dev(k), dev(v), Attn(keys=keys, splits=splits)))
    want = oracle.attention_direct(oracle.AttnProblem(q, k, v, key_mask=mask.astype(np.int32)))
    check("masked", got, tiles, want)
    assert not to_np(got)[1].any()


@pytest.mark.parametrize("splits", [None, 2, 5])
@pytest.mark.parametrize("d,h,hkv,t", [(64, 4, 4, 1), (64, 8, 2, 1), (128, 4, 2, 2), (48, 4, 4, 3)])
def test_a_cache_with_a_row_map_and_appended_rows(device, splits, d, h, hkv, t):
    """The reference's cache fixture (tk/src/test/unit/ops.rs:585-627): lanes mapped onto two cache rows of three
    layers, lengths tk, 1, 37, tk - 1, 0, the step's own rows scored after the cached ones, a count of them a lane."""
    b, rows, layers, tk, n = 5, 2, 3, 700, 3
    g = Lcg(40)
    q = g.bf16((b, t, h, d))
    k, v = g.bf16((rows, tk, layers * hkv, d)), g.bf16((rows, tk, layers * hkv, d))
    k_app, v_app = g.bf16((b, n, hkv, d)), g.bf16((b, n, hkv, d))
    lens, row_map, seen = np.array([tk, 1, 37, tk - 1, 0]), np.array([0, 1, 1, 0, 1]), np.array([3, 2, 1, 3, 2])
    dev = lambda x: bf16_tensor(x, device)
    ints = lambda a: torch.tensor(a, dtype=torch.int64, device=device)
    cache = Cache(hkv, hkv, ints(row_map), (dev(k_app), dev(v_app)), ints(seen))
    got, tiles = both_paths(lambda: svod_amd.attention(dev(q), dev(k), dev(v),
                                                       Attn(keys=KeyMask.lens(ints(lens)), splits=splits, cache=cache)))
    p = oracle.AttnProblem(q, k, v, key_lens=lens, cache=oracle.Cache(hkv, hkv, row_map, (k_app, v_app), seen))
    check("cache", got, tiles, oracle.attention_direct(p))


def test_f16_operands_and_a_negative_scale(device):
    b, t, tk, h, hkv, d = 2, 1, 500, 4, 2, 64
    g = Lcg(12)
    q, k, v = (oracle.round_f16(g.bf16(s)) for s in ((b, t, h, d), (b, tk, hkv, d), (b, tk, hkv, d)))
    dev = lambda x: torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.float16).to(device)
    for scale in (None, -0.2):
        got, tiles = both_paths(lambda: svod_amd.attention(dev(q), dev(k), dev(v), Attn(scale=scale, splits=2)))
        want = oracle.attention_direct(oracle.AttnProblem(q, k, v, scale=scale, bf16=False))
        check("f16", got, tiles, want)


def test_rows_past_a_length_are_never_read(device):
    """K and V rows at and past a lane's length may hold anything (a cache's unwritten tail): NaN there reaches nothing."""
    b, t, tk, h, hkv, d = 2, 1, 300, 4, 2, 64
    g = Lcg(8)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    lens = np.array([130, 300])
    kd, vd = bf16_tensor(k, device), bf16_tensor(v, device)
    kd[0, 130:], vd[0, 130:] = float("nan"), float("inf")
    got = svod_amd.attention(bf16_tensor(q, device), kd, vd,
                             Attn(keys=KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))))
    torch.cuda.synchronize()
    assert STREAMED in svod_amd.chosen() or "combine_splits" in svod_amd.chosen()
    want = oracle.attention_direct(oracle.AttnProblem(q, k, v, key_lens=lens))
    assert max_abs(to_np(got), want) < 2e-2


def test_five_rows_run_key_tiles(device):
    b, t, tk, h, hkv, d = 1, 5, 100, 2, 2, 64
    g = Lcg(2)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    dev = lambda x: bf16_tensor(x, device)
    svod_amd.attention(dev(q), dev(k), dev(v), Attn())
    assert STREAMED not in svod_amd.chosen()
    svod_amd.attention(dev(q[:, :1]), dev(k), dev(v), Attn(causal=True))
    assert STREAMED not in svod_amd.chosen()


def test_a_captured_decoder_step_replays(device):
    b, t, tk, h, hkv, d = 4, 1, 1000, 8, 8, 64
    g = Lcg(21)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    qd, kd, vd = (bf16_tensor(x, device) for x in (q, k, v))
    out = torch.empty_like(qd)
    ws = torch.empty(4 * b * t * h * (d + 2) * 4, dtype=torch.uint8, device=device)
    call = lambda: svod_amd.attention(qd, kd, vd, Attn(splits=4), out=out, workspace=ws)
    call()
    torch.cuda.synchronize()
    eager = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


def test_unasked_two_rows_stream_and_three_do_not(device):
    svod_amd.tune_decode(svod_amd.DECODE_ROWS_DEFAULT)
    g = Lcg(4)
    k, v = g.bf16((1, 100, 1, 64)), g.bf16((1, 100, 1, 64))
    dev = lambda x: bf16_tensor(x, device)
    for heads, streams in ((1, True), (2, True), (3, False)):
        svod_amd.attention(dev(g.bf16((1, 1, heads, 64))), dev(k), dev(v), Attn(splits=1))
        assert (STREAMED in svod_amd.chosen()) == streams, (heads, svod_amd.chosen())


def test_the_fused_projection_read_in_place(device):
    """attention_packed (tk/src/ops/attention.rs:104-122) on a decoder step: q, k and v are views of one row."""
    b, t, h, hkv, d = 3, 1, 4, 2, 64
    g = Lcg(6)
    qkv = g.bf16((b, t, (h + 2 * hkv) * d))
    qkv_d = bf16_tensor(qkv, device)
    got = svod_amd.attention_packed(qkv_d, h, hkv, Attn(splits=1))
    torch.cuda.synchronize()
    assert STREAMED in svod_amd.chosen(), svod_amd.chosen()
    q, k, v = (qkv[..., a * d:e * d].reshape(b, t, -1, d) for a, e in ((0, h), (h, h + hkv), (h + hkv, h + 2 * hkv)))
    want = oracle.attention_direct(oracle.AttnProblem(np.ascontiguousarray(q), np.ascontiguousarray(k), np.ascontiguousarray(v)))
    assert max_abs(to_np(got), want) < 2e-2


def test_a_bound_batch_runs_its_live_rows_only(device):
    b, live, t, tk, h, d = 4, 2, 1, 300, 4, 64
    g = Lcg(13)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, h, d)), g.bf16((b, tk, h, d))
    out = torch.full((b, t, h, d), 7.0, dtype=torch.bfloat16, device=device)
    svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device), Attn(splits=1, batch_live=live), out=out)
    torch.cuda.synchronize()
    assert STREAMED in svod_amd.chosen()
    want = oracle.attention_direct(oracle.AttnProblem(q[:live], k[:live], v[:live]))
    assert max_abs(to_np(out[:live]), want) < 2e-2
    assert (to_np(out[live:]) == 7.0).all()


def test_random_calls_agree_with_the_tile_kernel(device):
    """A seeded sweep over head sizes, row counts, GQA groups, key counts around the block edges, both types, split
    counts, every key-mask form, caches with row maps, layers and appended rows, and scales of either sign: the
    two kernels give the same outcome (a result or the same refusal) and results within the op's bar."""
    import random
    rng = random.Random(20)
    torch.manual_seed(20)
    compared = 0
    for case in range(160):
        d = rng.choice([32, 48, 64, 128, 256])
        rows = rng.choice([1, 1, 2, 2, 3, 4])
        group = rng.choice([g for g in (1, 2, 3, 4) if rows % g == 0])
        t, hkv = rows // group, rng.choice([1, 2, 3, 5, 8])
        h, b = hkv * group, rng.choice([1, 2, 3, 7, 16])
        tk = rng.choice([1, 5, 63, 64, 65, 127, 128, 129, 300, 777, 1500, 4096])
        dt = torch.float16 if rng.random() < 0.3 else torch.bfloat16
        splits = rng.choice([None, None, 1, 2, 3, 5, 9])
        kind = rng.choice(["none", "lens", "lens64", "mask", "maskint"])
        cached = rng.random() < 0.4
        layers = rng.choice([1, 3]) if cached else 1
        crow = rng.choice([b, max(1, b // 2), b + 2]) if cached else b
        mapped = cached and (crow != b or rng.random() < 0.5)
        if cached and not mapped and crow != b:
            crow = b
        q = torch.randn(b, t, h, d, device=device).to(dt)
        k = torch.randn(crow, tk, layers * hkv, d, device=device).to(dt)
        v = torch.randn(crow, tk, layers * hkv, d, device=device).to(dt)
        keys = KeyMask.none()
        if kind in ("lens", "lens64"):
            lens = [rng.choice([0, 1, tk, tk // 2, max(tk - 1, 0), rng.randint(0, tk)]) for _ in range(b)]
            keys = KeyMask.lens(torch.tensor(lens, dtype=torch.int64 if kind == "lens64" else torch.int32, device=device))
        elif kind in ("mask", "maskint"):
            m = torch.rand(b, tk, device=device) < rng.choice([0.1, 0.5, 0.9])
            if b > 1:
                m[1] = False
            keys = KeyMask.bool(m if kind == "mask" else m.to(torch.int32))
        cache = None
        if cached:
            app = rng.choice([0, 1, 3, 8])
            appended = (torch.randn(b, app, hkv, d, device=device).to(dt), torch.randn(b, app, hkv, d, device=device).to(dt)) if app else None
            app_lens = (torch.tensor([rng.randint(0, app) for _ in range(b)], dtype=torch.int32, device=device)
                        if app and rng.random() < 0.5 else None)
            row_map = (torch.tensor([rng.randrange(crow) for _ in range(b)], dtype=rng.choice([torch.int32, torch.int64]), device=device)
                       if mapped else None)
            cache = Cache((layers - 1) * hkv, hkv, row_map, appended, app_lens)
        opts = Attn(keys=keys, splits=splits, cache=cache, scale=rng.choice([None, None, 0.07, -0.1]))
        name = f"case {case}: b{b} t{t} tk{tk} h{h}/{hkv} d{d} {dt} splits={splits} {kind} cached={cached} layers={layers} mapped={mapped}"
        outcomes = []
        for knob in (4, 0):
            svod_amd.tune_decode(knob)
            try:
                ws = torch.empty(16 * b * t * h * (d + 2) * 4, dtype=torch.uint8, device=device)
                outcomes.append(svod_amd.attention(q, k, v, opts, workspace=ws))
            except (svod_amd.OpError, svod_amd.GraphFallback) as e:
                outcomes.append(type(e).__name__ + ": " + str(e))
        svod_amd.tune_decode(4)
        torch.cuda.synchronize()
        one, two = outcomes
        if isinstance(one, str) or isinstance(two, str):
            assert one == two, name
            continue
        compared += 1
        assert torch.isfinite(one.float()).all(), name
        if one.numel():
            assert float((one.float() - two.float()).abs().max()) < 2e-2, name
    assert compared > 120
