"""Grouped tiles: a decoder step under GQA (heads / kv_heads * T <= 128, no causal or per-row mask) runs the
heads of a KV head's group side by side in one query tile, so the group shares one pass over its K and V.
A row's arithmetic does not depend on the tile it sits in: the output is bit-equal to the same call with
the KV heads repeated per query head (plain multi-head attention, which takes the ungrouped path)."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Attn, Cache, KeyMask
from util import Lcg, bf16_tensor, bits, max_abs, to_np

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("key_tiles")]

# (name, b, t, tk, h, hkv, d, splits, lens, biased)
CASES = [
    ("one query, group of four", 3, 1, 500, 8, 2, 64, None, [500, 77, 0], False),
    ("one query, group of eight, d128, long keys (split unasked)", 2, 1, 4096, 16, 2, 128, None, None, False),
    ("sixteen queries, group of eight: a full tile", 2, 16, 300, 8, 1, 64, None, [300, 129], False),
    ("five queries, group of three, biased", 2, 5, 200, 6, 2, 64, None, [200, 64], True),
    ("three splits named", 1, 2, 1000, 8, 2, 64, 3, None, False),
    ("seven queries, group of two, d128", 4, 7, 130, 4, 2, 128, None, [130, 1, 64, 65], False),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,splits,lens,biased", CASES, ids=[c[0] for c in CASES])
def test_grouped_tiles_match_repeated_kv_heads_bit_for_bit(device, name, b, t, tk, h, hkv, d, splits, lens, biased):
    g = Lcg(31)
    q, k, v = g.bf16((b, t, h, d)), g.bf16((b, tk, hkv, d)), g.bf16((b, tk, hkv, d))
    bias = g.bf16((b, h, t, tk), mul=2.0) if biased else None
    keys = KeyMask.none() if lens is None else KeyMask.lens(torch.tensor(lens, dtype=torch.int32, device=device))
    dev = lambda x: None if x is None else bf16_tensor(x, device)
    # Splits are pinned so that both calls run the same ones (unasked, the rule counts workgroups).
    ws_q, ws_k = svod_amd.ops._desc(dev(q)), svod_amd.ops._desc(dev(k))
    opts = Attn(keys=keys, splits=splits, bias=dev(bias))
    grouped = svod_amd.attention(dev(q), dev(k), dev(v), opts)
    chosen = svod_amd.chosen()
    used = splits or (1 if "combine_splits" not in chosen else None)
    if used is None:  # the rule split it: ask how many ways, and name that count for the repeated call
        import ctypes
        a = svod_amd.ops._attn_options(Attn(keys=keys), [])
        need = svod_amd.load_library().svodk_attention_workspace(ctypes.byref(ws_q), ctypes.byref(ws_k), ctypes.byref(a))
        used = need // (b * t * h * (d + 2) * 4)
        assert used > 1
    group = h // hkv
    plain = svod_amd.attention(dev(q), dev(np.repeat(k, group, axis=2)), dev(np.repeat(v, group, axis=2)),
                               Attn(keys=keys, splits=used, bias=dev(bias)))
    torch.cuda.synchronize()
    assert np.array_equal(bits(grouped), bits(plain))
    want = oracle.attention_direct(oracle.AttnProblem(q, k, v, key_lens=None if lens is None else np.asarray(lens), bias=bias))
    assert max_abs(to_np(grouped), want) < 2e-2


@pytest.mark.parametrize("splits", [None, 2, 5])
def test_a_grouped_decoder_step_over_a_cache_with_appended_rows(device, splits):
    b, rows, layers, t, d, h, hkv, tk, n = 4, 2, 2, 1, 64, 8, 2, 700, 1
    g = Lcg(9)
    q = g.bf16((b, t, h, d))
    k, v = g.bf16((rows, tk, layers * hkv, d)), g.bf16((rows, tk, layers * hkv, d))
    k_app, v_app = g.bf16((b, n, hkv, d)), g.bf16((b, n, hkv, d))
    lens, row_map = np.array([700, 1, 333, 0]), np.array([1, 0, 0, 1])
    dev = lambda x: bf16_tensor(x, device)
    ints = lambda a: torch.tensor(a, dtype=torch.int32, device=device)
    got = svod_amd.attention(dev(q), dev(k), dev(v), Attn(keys=KeyMask.lens(ints(lens)), splits=splits,
                             cache=Cache(hkv, hkv, ints(row_map), (dev(k_app), dev(v_app)))))
    torch.cuda.synchronize()
    p = oracle.AttnProblem(q, k, v, key_lens=lens, cache=oracle.Cache(hkv, hkv, row_map, (k_app, v_app)))
    assert max_abs(to_np(got), oracle.attention_direct(p)) < 2e-2
