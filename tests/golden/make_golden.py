#!/usr/bin/env python3
"""Writes the golden fixtures of this directory.

Inputs come from the reference's own test generators (the 64-bit LCG of
tk/src/test/unit/mod.rs:442-450 and the mask formulas of tk/src/test/unit/attention.rs:69-81,
tk/src/test/unit/heads.rs:37-56).  Expected outputs come from routines that are neither the
oracle nor the reference: ``torch.nn.functional.scaled_dot_product_attention`` in float64 for
attention, and a numpy float64 evaluation written here for the prologue.  Nothing is read from
the reference checkout; the fixtures pin the oracle (CPU tests) and the HIP kernels (GPU tests).

    python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
A, C, MASK = 6364136223846793005, 1442695040888963407, (1 << 64) - 1


def lcg(seed, n):
    """Pure-Python big-integer evaluation of the reference LCG: n draws on [-1, 1)."""
    out = np.empty(n, dtype=np.float64)
    for i in range(n):
        seed = (seed * A + C) & MASK
        out[i] = (seed >> 33) / float(1 << 31) * 2.0 - 1.0
    return out, seed


def bf16(x):
    """Round to bf16 through torch (an independent implementation of nearest-even)."""
    return torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).to(torch.float32).numpy()


def sdpa64(q, k, v, keep, scale):
    """q [B,T,H,D], k/v [B,Tk,Hkv,D], keep [B,T,Tk] bool -> [B,T,H,D] float64 (zeros where no key)."""
    b, t, h, d = q.shape
    hkv = k.shape[2]
    qt = torch.from_numpy(q).double().permute(0, 2, 1, 3)
    kt = torch.from_numpy(k).double().permute(0, 2, 1, 3).repeat_interleave(h // hkv, dim=1)
    vt = torch.from_numpy(v).double().permute(0, 2, 1, 3).repeat_interleave(h // hkv, dim=1)
    m = torch.from_numpy(keep)[:, None, :, :]
    o = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=m, scale=scale)
    o = torch.where(m.any(dim=-1, keepdim=True), o, torch.zeros_like(o))  # a row no key reaches is zeros
    return o.permute(0, 2, 1, 3).contiguous().numpy()


def attention_fixture(name, b, t, tk, h, hkv, d, causal, lens, key_mask, seed=5, scale=None):
    n_q, n_k = b * t * h * d, b * tk * hkv * d
    x, seed = lcg(seed, n_q)
    q = bf16(x).reshape(b, t, h, d)
    x, seed = lcg(seed, n_k)
    k = bf16(x).reshape(b, tk, hkv, d)
    x, seed = lcg(seed, n_k)
    v = bf16(x).reshape(b, tk, hkv, d)
    keep = np.ones((b, t, tk), dtype=bool)
    if causal:
        keep &= (np.arange(tk)[None, :] <= np.arange(t)[:, None])[None]
    lens_a = None
    if lens is not None:
        lens_a = np.asarray(lens, dtype=np.int32)
        keep &= (np.arange(tk)[None, None, :] < lens_a[:, None, None])
    mask_a = None
    if key_mask:
        bb, jj = np.meshgrid(np.arange(b), np.arange(tk), indexing="ij")
        mask_a = (bb + jj) % 5 != 2
        keep &= mask_a[:, None, :]
    scale = scale if scale is not None else float(np.float32(1.0) / np.sqrt(np.float32(d)))
    out = sdpa64(q, k, v, keep, scale)
    arrays = dict(q=q, k=k, v=v, out=out, keep=keep, causal=np.array(causal), scale=np.array(scale, dtype=np.float32))
    if lens_a is not None:
        arrays["lens"] = lens_a
    if mask_a is not None:
        arrays["key_mask"] = mask_a
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)


def heads_fixture(name, b, t, h, hkv, d, seed=7):
    """heads.rs `inputs(seed 7)`: qkv = 3x, weights 1 + 0.5x, angles row*0.01*(1+col); f64 expected."""
    slots, half = h + 2 * hkv, d // 2
    x, seed = lcg(seed, b * t * slots * d)
    qkv = bf16(3.0 * x).reshape(b, t, slots, d)
    x, seed = lcg(seed, d)
    q_w = bf16(1.0 + 0.5 * x)
    x, seed = lcg(seed, d)
    k_w = bf16(1.0 + 0.5 * x)
    e = np.arange(t * half)
    ang = (e // half).astype(np.float64) * 0.01 * (1.0 + (e % half).astype(np.float64))
    cos, sin = bf16(np.cos(ang)).reshape(t, half), bf16(np.sin(ang)).reshape(t, half)
    eps = 1e-6

    def path(xs, w, rotate):
        xs = xs.astype(np.float64)
        if w is not None:
            inv = 1.0 / np.sqrt((xs * xs).mean(axis=-1, keepdims=True) + eps)
            xs = xs * inv * w.astype(np.float64)
        if rotate:
            c, s = cos.astype(np.float64)[None, :, None, :], sin.astype(np.float64)[None, :, None, :]
            x1, x2 = xs[..., :half], xs[..., half:]
            xs = np.concatenate([x1 * c - x2 * s, x1 * s + x2 * c], axis=-1)
        return xs

    q = path(qkv[:, :, :h], q_w, True)
    k = path(qkv[:, :, h:h + hkv], k_w, True)
    v = qkv[:, :, h + hkv:].astype(np.float64)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), qkv=qkv.reshape(b, t, slots * d), q_w=q_w, k_w=k_w, cos=cos,
                        sin=sin, q=q, k=k, v=v, eps=np.array(eps), dims=np.array([h, hkv, d]))


def config1_fixture():
    """Config 1 of the benchmark: fp32 B1 H1 S128 D64 N(0,1) from the shared generator, f64 expected."""
    import sys
    sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
    from svod_amd import workloads as W

    w = W.config1()
    q, k, v = (x.numpy() for x in (w.q, w.k, w.v))
    keep = np.ones((1, 128, 128), dtype=bool)
    np.savez_compressed(os.path.join(HERE, "config1_fp32.npz"), q=q, k=k, v=v, out=sdpa64(q, k, v, keep, 0.125),
                        scale=np.array(0.125, dtype=np.float32))


def bf16_kat_fixture():
    """The rounding known answers of tk/src/test/unit/interp.rs:197-216 (value, nearest, toward zero)
    plus the bit-level rule on a sweep of patterns, rounded by torch."""
    rows = [(1.0 + 3.0 / 512.0, 1.0 + 1.0 / 128.0, 1.0), (-(1.0 + 3.0 / 512.0), -(1.0 + 1.0 / 128.0), -1.0),
            (0.5, 0.5, 0.5), (0.0, 0.0, 0.0)]
    rng = np.random.default_rng(0)
    pats = rng.integers(0, 1 << 32, size=4096, dtype=np.uint64).astype(np.uint32)
    ties = (rng.integers(0, 1 << 16, size=512, dtype=np.uint64).astype(np.uint32) << 16) | 0x8000  # exact halves
    pats = np.concatenate([pats, ties])
    vals = pats.view(np.float32)
    ok = np.isfinite(vals)
    vals = vals[ok]
    np.savez_compressed(os.path.join(HERE, "bf16_rounding.npz"), kat=np.array(rows, dtype=np.float64), sweep=vals,
                        sweep_rounded=bf16(vals))


if __name__ == "__main__":
    attention_fixture("attn_plain_64x96_d64", 2, 64, 96, 2, 2, 64, False, None, False)
    attention_fixture("attn_causal_64x96_d64", 2, 64, 96, 2, 2, 64, True, None, False)
    attention_fixture("attn_lens_64x96_d64", 2, 64, 96, 2, 2, 64, False, [96, 7], False)
    attention_fixture("attn_keymask_64x96_d64", 2, 64, 96, 2, 2, 64, False, None, True)
    attention_fixture("attn_causal_lens_gqa_64x96_d128", 2, 64, 96, 4, 2, 128, True, [90, 50], False)
    attention_fixture("attn_nokeys_64x96_d64", 2, 64, 96, 2, 2, 64, False, [96, 0], False)
    heads_fixture("heads_9rows_4q2kv_d64", 2, 9, 4, 2, 64)
    heads_fixture("heads_10rows_4q2kv_d128", 1, 10, 4, 2, 128)
    config1_fixture()
    bf16_kat_fixture()
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
