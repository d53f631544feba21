"""Attention over a cache (Cache of tk/src/ops/attention.rs:39-56; tk/src/kernels/attention.rs:544-550,
739-755, 827-846): k and v hold several layers' heads, batch lanes map to cache rows, and the rows a decoder
step has just projected are scored after the cached prefix.  The cases are the reference's own
(tk/src/test/unit/ops.rs:585-627: five lanes over two cache rows of three layers, lengths tk, 1, 37, tk-1, 0)
at the head sizes this library has kernels for."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, Cache, KeyMask
from util import Lcg, assert_bf16_parity, bf16_tensor, bits, max_abs, to_np

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("key_tiles")]

B, ROWS, LAYERS = 5, 2, 3


def operands(t, d, h, tk, appended, seed=40):
    g = Lcg(seed)
    q = g.bf16((B, t, h, d))
    k, v = g.bf16((ROWS, tk, LAYERS * h, d)), g.bf16((ROWS, tk, LAYERS * h, d))
    k_app, v_app = g.bf16((B, appended, h, d)), g.bf16((B, appended, h, d))
    bias = g.bf16((B, h, t, tk + appended), mul=2.0)
    lens = np.array([tk, 1, 37, tk - 1, 0])
    row_map = np.array([0, 1, 1, 0, 1])
    seen = np.array([max(appended - lane % 3, 1) for lane in range(B)])
    return q, k, v, k_app, v_app, bias, lens, row_map, seen


def run(device, t, d, h, tk, splits, appended, counted, biased, int_dtype=torch.int32, mapped=True):
    q, k, v, k_app, v_app, bias, lens, row_map, seen = operands(t, d, h, tk, appended)
    if not mapped:
        k, v = (np.ascontiguousarray(x[row_map]) for x in (k, v))  # a cache row a lane
    ints = lambda a: torch.from_numpy(np.asarray(a)).to(int_dtype).to(device)
    cache = Cache(head_start=h, kv_heads=h, row_map=ints(row_map) if mapped else None,
                  appended=(bf16_tensor(k_app, device), bf16_tensor(v_app, device)),
                  app_lens=ints(seen) if counted else None)
    opts = Attn(keys=KeyMask.lens(ints(lens)), cache=cache, splits=splits,
                bias=bf16_tensor(bias, device) if biased else None)
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device), opts)
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, k, v, key_lens=lens, bias=bias if biased else None,
                           cache=oracle.Cache(h, h, row_map if mapped else None, (k_app, v_app), seen if counted else None))
    return got, p


# ([t, d, h, tk], splits, appended, counted, biased): ops.rs:585-591 (the d 48 cases also at 64)
CASES = [
    ("a streaming chunk: eight queries, eight appended, d 48", [8, 48, 16, 128], None, 8, False, False),
    ("sixteen counted appended, two splits, d 48", [16, 48, 16, 128], 2, 16, True, False),
    ("one query, 1500 keys, four splits", [1, 64, 20, 1500], 4, 1, False, False),
    ("d 128 unsplit", [1, 128, 8, 300], None, 1, False, False),
    ("three queries, two splits", [3, 64, 4, 200], 2, 1, False, False),
    ("biased, three queries, two splits", [3, 64, 4, 200], 2, 1, False, True),
    ("a streaming chunk: eight queries, eight appended", [8, 64, 16, 128], None, 8, False, False),
    ("sixteen counted appended, two splits", [16, 64, 16, 128], 2, 16, True, False),
    ("biased, counted appended", [8, 64, 4, 128], None, 8, True, True),
    ("a full block of appended rows, d 128, biased", [5, 128, 4, 333], None, 64, True, True),
    ("many queries over a long cache", [200, 64, 4, 700], None, 3, True, False),
]


@pytest.mark.parametrize("name,dims,splits,appended,counted,biased", CASES, ids=[c[0] for c in CASES])
def test_cached_attention_matches_a_direct_softmax(device, name, dims, splits, appended, counted, biased):
    t, d, h, tk = dims
    got, p = run(device, t, d, h, tk, splits, appended, counted, biased)
    direct = oracle.attention_direct(p)
    program = oracle.attention_flash(p, bq=128, bkv=64, splits=min(splits or 1, (tk + 63) // 64))
    assert_bf16_parity(name, to_np(got), direct, program)


def test_a_lane_with_no_cached_keys_sees_only_the_appended_rows(device):
    """Lane 4 of the fixture has length 0: its output is the softmax over its appended rows alone."""
    t, d, h, tk, appended = 3, 64, 4, 200, 4
    got, p = run(device, t, d, h, tk, None, appended, False, False)
    q, k_app, v_app = p.q[4], p.cache.appended[0][4], p.cache.appended[1][4]
    s = np.einsum("thd,nhd->htn", q.astype(np.float64), k_app.astype(np.float64)) / np.sqrt(d)
    w = np.exp(s - s.max(-1, keepdims=True))
    w /= w.sum(-1, keepdims=True)
    want = np.einsum("htn,nhd->thd", w, v_app.astype(np.float64))
    assert max_abs(to_np(got)[4], want) < 2e-2


def test_the_row_map_is_a_gather_and_its_integers_may_be_64_bit(device):
    t, d, h, tk = 5, 64, 4, 150
    mapped, _ = run(device, t, d, h, tk, None, 2, True, False)
    wide, _ = run(device, t, d, h, tk, None, 2, True, False, int_dtype=torch.int64)
    gathered, _ = run(device, t, d, h, tk, None, 2, True, False, mapped=False)
    assert np.array_equal(bits(mapped), bits(wide))
    assert np.array_equal(bits(mapped), bits(gathered))


def test_a_cache_without_appended_rows_is_a_view_of_its_heads(device):
    """head_start and kv_heads alone: the same bits as attention over the narrowed, gathered tensors."""
    t, d, h, tk = 40, 64, 4, 300
    q, k, v, _, _, _, lens, row_map, _ = operands(t, d, h, tk, 1)
    dev = lambda x: bf16_tensor(x, device)
    ints = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    for causal in (False, True):
        cached = svod_amd.attention(dev(q), dev(k), dev(v), Attn(causal=causal, keys=KeyMask.lens(ints(lens)),
                                                                 cache=Cache(2 * h, h, row_map=ints(row_map))))
        plain = svod_amd.attention(dev(q), dev(np.ascontiguousarray(k[row_map][:, :, 2 * h:3 * h])),
                                   dev(np.ascontiguousarray(v[row_map][:, :, 2 * h:3 * h])),
                                   Attn(causal=causal, keys=KeyMask.lens(ints(lens))))
        assert np.array_equal(bits(cached), bits(plain))


def test_a_mapped_row_outside_the_cache_reads_its_nearest_row(device):
    """The map is device data no host check sees: rows past the cache's ends are held inside it, so a
    bad map gives the result of a clamped one instead of a read of memory that is not there."""
    t, d, h, tk = 40, 64, 4, 300
    q, k, v, _, _, _, lens, _, _ = operands(t, d, h, tk, 1)
    dev = lambda x: bf16_tensor(x, device)
    ints = lambda a, dt=torch.int32: torch.tensor(a, dtype=dt, device=device)
    rows = k.shape[0]
    wild = np.array([-3, rows, 0, 2 ** 31 - 1, rows - 1][:B] + [0] * max(0, B - 5))
    tame = np.clip(wild, 0, rows - 1)
    for dt in (torch.int32, torch.int64):
        got = svod_amd.attention(dev(q), dev(k), dev(v), Attn(keys=KeyMask.lens(ints(lens)),
                                                             cache=Cache(2 * h, h, row_map=ints(wild, dt))))
        want = svod_amd.attention(dev(q), dev(k), dev(v), Attn(keys=KeyMask.lens(ints(lens)),
                                                              cache=Cache(2 * h, h, row_map=ints(tame, dt))))
        assert np.array_equal(bits(got), bits(want))


def test_what_the_cache_has_no_kernel_for_keeps_the_graph(device):
    t, d, h, tk = 4, 64, 4, 100
    q, k, v, _, _, _, lens, row_map, _ = operands(t, d, h, tk, 1)
    dev = lambda x: bf16_tensor(x, device)
    ints = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    g = Lcg(3)
    many = (dev(g.bf16((B, 65, h, d))), dev(g.bf16((B, 65, h, d))))
    for opts in (Attn(keys=KeyMask.lens(ints(lens)), cache=Cache(h, h, ints(row_map), appended=many)),):
        with pytest.raises(svod_amd.GraphFallback) as e:
            svod_amd.attention(dev(q), dev(k), dev(v), opts)
        assert e.value.why == svod_amd.Fallback.Config


# A cache under per-row key ranges: Attn allows every combination (tk/src/ops/attention.rs:60-86); the ranges
# hide cached keys only and the appended rows answer to their own count (tk/src/test/unit/attention.rs:138-141).
# (name, [t, d, h, tk], masks, appended, counted, biased, splits)
RANGED = [
    ("a causal window over a cache", [96, 64, 4, 200], dict(causal=True, window=(40, 0)), 0, False, False, None),
    ("a window, eight appended rows", [8, 64, 4, 300], dict(window=(100, 150)), 8, True, False, None),
    ("chunks of 16 behind a streaming chunk of queries, d 128", [16, 128, 4, 333], dict(chunk=(16, 4, 0)), 16, True, False, None),
    ("segment starts, biased", [40, 64, 4, 128], dict(seg=20), 3, False, True, None),
    ("every mask at once, d 48", [64, 48, 4, 128], dict(causal=True, window=(50, 0), chunk=(32, 3, 0), seg=40), 8, True, False, None),
    ("a window with named splits runs the splits", [4, 64, 4, 640], dict(window=(600, 600)), 4, True, False, 2),
]


@pytest.mark.parametrize("name,dims,masks,appended,counted,biased,splits", RANGED, ids=[c[0] for c in RANGED])
def test_a_cache_under_per_row_ranges(device, name, dims, masks, appended, counted, biased, splits):
    t, d, h, tk = dims
    q, k, v, k_app, v_app, bias, lens, row_map, seen = operands(t, d, h, tk, max(appended, 1))
    lens = np.array([tk, 1, 37, tk - 1, 0])
    masks = dict(masks)
    seg = None
    if "seg" in masks:
        n = masks.pop("seg")
        seg = np.tile(np.arange(t) - np.arange(t) % n, (B, 1))
    if appended == 0:
        bias = np.ascontiguousarray(bias[..., :tk])
    ints = lambda a: torch.from_numpy(np.asarray(a)).to(torch.int32).to(device)
    app = (bf16_tensor(k_app, device), bf16_tensor(v_app, device)) if appended else None
    cache = Cache(head_start=h, kv_heads=h, row_map=ints(row_map), appended=app,
                  app_lens=ints(seen) if counted and appended else None)
    opts = Attn(causal=masks.get("causal", False), window=masks.get("window"), chunk=masks.get("chunk"),
                seg_start=ints(seg) if seg is not None else None, keys=KeyMask.lens(ints(lens)), cache=cache,
                splits=splits, bias=bf16_tensor(bias, device) if biased else None)
    got = svod_amd.attention(bf16_tensor(q, device), bf16_tensor(k, device), bf16_tensor(v, device), opts)
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    p = oracle.AttnProblem(q, k, v, causal=masks.get("causal", False), window=masks.get("window"), chunk=masks.get("chunk"),
                           seg_start=seg, key_lens=lens, bias=bias if biased else None,
                           cache=oracle.Cache(h, h, row_map, (k_app, v_app) if appended else None,
                                              seen if counted and appended else None))
    direct = oracle.attention_direct(p)
    program = oracle.attention_flash(p, bq=128, bkv=64, splits=min(splits or 1, (tk + 63) // 64))
    assert_bf16_parity(name, to_np(got), direct, program)
    # Rows no key reaches (a lane without cached keys and without visible appended rows) are zeros.
    assert np.isfinite(to_np(got)).all()


@pytest.mark.parametrize("splits", [None, 4], ids=["whole", "a decoder step over four splits"])
def test_a_non_finite_unread_element_never_reaches_the_output(device, splits):
    """attention.rs:572-592: the cache's first row, which no lane's map reaches, and every row past a
    lane's keys hold an infinity and NaNs, as memory nothing initialised may; the last key block is
    partial.  The kernel reads zeros past the keys and never the unmapped row: same bits as with clean memory."""
    t, d, h, tk = 1, 64, 4, 100
    q, k, v, _, _, _, _, _, _ = operands(t, d, h, tk, 1)
    lens = np.array([100, 37, 1, 99, 64])
    row_map = np.ones(B, dtype=np.int64)
    dev = lambda x: bf16_tensor(x, device)
    ints = lambda a: torch.tensor(a, dtype=torch.int32, device=device)

    def call(kk, vv):
        out = svod_amd.attention(dev(q), dev(kk), dev(vv), Attn(keys=KeyMask.lens(ints(lens)), splits=splits,
                                                              cache=Cache(h, h, row_map=ints(row_map))))
        torch.cuda.synchronize()
        return out

    clean = call(k, v)
    k2, v2 = k.copy(), v.copy()
    for x in (k2, v2):
        x[0] = np.nan
        x[0, 0, 0, 0] = np.inf
        x[1, 37:, :h] = np.nan      # heads before the launch's and rows past the shortest lane's keys:
        x[1, 100:] = np.inf         # the longest lane sees rows 0..99 of heads h..2h-1 only
    k2[1, :100, h:2 * h], v2[1, :100, h:2 * h] = k[1, :100, h:2 * h], v[1, :100, h:2 * h]
    dirty = call(k2, v2)
    assert np.isfinite(to_np(dirty)).all()
    assert np.array_equal(bits(dirty), bits(clean))


def test_a_cache_whose_rows_span_more_than_two_gib(device):
    """A decoder step over a cache row of 64 KiB a token (512 heads of 64 over every layer) and 40 000 tokens: one
    (lane, head)'s keys span 2.6 GB, past what 32-bit byte offsets reach; the fills count from each key block's own
    64-bit base.  Two lanes over two rows, the layer's four heads near the end of the row, key lengths in the far part."""
    rows, tk, all_heads, h, d, start = 2, 40_000, 512, 4, 64, 500
    g = torch.Generator(device=device).manual_seed(3)
    k = torch.randn((rows, tk, all_heads, d), generator=g, device=device, dtype=torch.bfloat16)
    v = torch.randn((rows, tk, all_heads, d), generator=g, device=device, dtype=torch.bfloat16)
    q = torch.randn((rows, 1, h, d), generator=g, device=device, dtype=torch.bfloat16)
    lens = np.array([tk, 33_333])
    got = svod_amd.attention(q, k, v, Attn(keys=KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device)),
                                           cache=Cache(head_start=start, kv_heads=h)))
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "attention"'), svod_amd.chosen()
    ks, vs = (to_np(x[:, :, start:start + h].contiguous()) for x in (k, v))
    want = oracle.attention_direct(oracle.AttnProblem(to_np(q), ks, vs, key_lens=lens))
    assert max_abs(to_np(got), want) < 2e-2
