"""Parity of the HIP prologue (through the C ABI) with the CPU oracle.

Cases follow tk/src/test/unit/heads.rs:112-161 and tk/src/test/unit/ops.rs:645-672."""
import numpy as np
import pytest
import torch

import oracle
import svod_amd
from svod_amd import Qkv
from util import Lcg, bf16_tensor, bits, max_abs, to_np

pytestmark = pytest.mark.gpu


def reference_inputs(batch, t, heads, kv_heads, d, norms, rope, seed):
    """``inputs()`` of heads.rs:37-56: qkv = 3x, w = 1 + 0.5x, angles row·0.01·(1 + col)."""
    g = Lcg(seed)
    slots, half = heads + 2 * kv_heads, d // 2
    qkv = g.bf16((batch, t, slots * d), mul=3.0)
    q_w = g.bf16((d,), mul=0.5, add=1.0) if norms[0] else None
    k_w = g.bf16((d,), mul=0.5, add=1.0) if norms[1] else None
    cos = sin = None
    if rope is not None:
        rows = batch * t if rope else t
        e = np.arange(rows * half)
        ang = (e // half).astype(np.float64) * 0.01 * (1.0 + (e % half).astype(np.float64))
        shape = (batch if rope else 1, t, 1, half)
        cos = oracle.round_bf16(np.cos(ang).astype(np.float32)).reshape(shape)
        sin = oracle.round_bf16(np.sin(ang).astype(np.float32)).reshape(shape)
    return qkv, q_w, k_w, cos, sin


def run(device, qkv, heads, kv_heads, d, q_w, k_w, cos, sin, eps=1e-6, batch_live=None, out=None):
    t = lambda a: None if a is None else bf16_tensor(a, device)
    opts = Qkv(heads=heads, kv_heads=kv_heads, head_dim=d, q_norm=t(q_w), k_norm=t(k_w), eps=eps,
               rope=None if cos is None else (t(cos), t(sin)), batch_live=batch_live)
    q, k, v = svod_amd.heads(t(qkv), opts, out=out)
    torch.cuda.synchronize()
    assert svod_amd.chosen().startswith('Kernel { op: "heads", family: "heads"'), svod_amd.chosen()
    return q, k, v


# (name, batch, t, heads, kv_heads, d, norms, rope: None | False (by position) | True (by token))
CASES = [
    ("normed and rotated, shared tables", 2, 9, 4, 2, 64, (True, True), False),
    ("d 128, tables per batch", 2, 10, 4, 2, 128, (True, True), True),
    ("rotated only", 2, 5, 2, 2, 64, (False, False), False),
    ("q normed only", 2, 8, 4, 1, 64, (True, False), None),
    ("a split", 2, 3, 2, 1, 32, (False, False), None),
    ("d 64, partial block", 2, 37, 4, 2, 64, (True, True), False),
    ("d 128, 8 over 2, by token", 2, 40, 8, 2, 128, (True, True), True),
    ("a split, d 64", 2, 16, 2, 2, 64, (False, False), None),
    ("d 16", 1, 7, 2, 1, 16, (True, True), False),
    ("d 256", 2, 11, 2, 2, 256, (True, True), False),
    ("k normed only, rotated", 3, 9, 4, 4, 64, (False, True), False),
]


@pytest.mark.parametrize("name,batch,t,heads,kv_heads,d,norms,rope", CASES, ids=[c[0] for c in CASES])
def test_heads_match_the_reference(device, name, batch, t, heads, kv_heads, d, norms, rope):
    qkv, q_w, k_w, cos, sin = reference_inputs(batch, t, heads, kv_heads, d, norms, rope, seed=11)
    got = run(device, qkv, heads, kv_heads, d, q_w, k_w, cos, sin)
    p = oracle.HeadsProblem(qkv, heads, kv_heads, d, q_w, k_w, 1e-6, cos, sin)
    direct = oracle.heads_direct(p)
    program = oracle.heads_kernel(p)
    graph = oracle.heads_graph(p)
    for i, what in enumerate("qkv"):
        g = to_np(got[i])
        assert np.isfinite(g).all()
        assert max_abs(g, direct[i]) <= 2e-2, what  # heads.rs:124
        assert max_abs(g, program[i]) <= 1e-2, what  # heads.rs:159
        # ops.rs:668-670: q and k within 2e-2 of the graph (rel, floor 1), v exactly.
        diff = np.abs(g.astype(np.float64) - graph[i])
        assert (diff <= 2e-2 * np.maximum(np.abs(graph[i]), 1.0)).all(), what
    # v is a copy: the same bits as the input's v slots.
    slots = heads + 2 * kv_heads
    want_v = bf16_tensor(qkv.reshape(batch, t, slots, d)[:, :, heads + kv_heads:, :], "cpu")
    assert np.array_equal(bits(got[2]), bits(want_v))
    # A slot with neither norm nor rope is a copy too.
    if not norms[0] and rope is None:
        want_q = bf16_tensor(qkv.reshape(batch, t, slots, d)[:, :, :heads, :], "cpu")
        assert np.array_equal(bits(got[0]), bits(want_q))


def test_only_the_live_batch_runs(device):
    """heads.rs:128-136: rows of a batch past the live bound are never written."""
    batch, t, heads, kv_heads, d = 2, 6, 2, 2, 64
    qkv, q_w, k_w, cos, sin = reference_inputs(batch, t, heads, kv_heads, d, (True, True), True, seed=3)
    mk = lambda n: torch.full((batch, t, n, d), float("nan"), dtype=torch.bfloat16, device=device)
    out = (mk(heads), mk(kv_heads), mk(kv_heads))
    q, k, v = run(device, qkv, heads, kv_heads, d, q_w, k_w, cos, sin, batch_live=1, out=out)
    for x in (q, k, v):
        g = to_np(x)
        assert np.isfinite(g[0]).all() and (g[0] != 0).any()
        assert np.isnan(g[1]).all()


def test_the_mean_square_of_a_normed_head_is_the_weights(device):
    """RMSNorm with unit weights leaves each head with mean square 1 (up to eps and bf16)."""
    batch, t, heads, kv_heads, d = 1, 33, 4, 2, 128
    qkv = Lcg(9).bf16((batch, t, (heads + 2 * kv_heads) * d), mul=5.0)
    ones = np.ones(d, dtype=np.float32)
    q, k, _ = run(device, qkv, heads, kv_heads, d, ones, ones, None, None)
    for x in (q, k):
        ms = (to_np(x).astype(np.float64) ** 2).mean(axis=-1)
        assert np.abs(ms - 1.0).max() < 1e-2
