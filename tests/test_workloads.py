"""The seeded benchmark inputs: the vectorised generator is the reference LCG bit for bit."""
import numpy as np
import torch

import oracle
from svod_amd import workloads as W


def test_the_vectorised_lcg_is_the_reference_lcg():
    n = (1 << 20) + 12345  # crosses a jump-table chunk
    got = W.lcg_uniform(n, 0x5EED0021).numpy()
    want, _ = oracle.lcg_fill(n, 0x5EED0021, bf16=False)
    assert np.array_equal(got.astype(np.float32), want)


def test_normals_agree_with_the_scalar_box_muller():
    got = W.normal(100001, 77, 0.5).to(torch.float32).numpy()
    want, _ = oracle.normal_fill(100001, 77, 0.5, bf16=False)
    assert np.abs(got - want).max() <= 1e-6
    assert abs(float(got.std()) - 0.5) < 5e-3 and abs(float(got.mean())) < 5e-3


def test_config_shapes_and_work_counts():
    w = W.config2(batch=4, seq=128)
    assert w.q.shape == (4, 128, 16, 64) and w.q.dtype == torch.bfloat16
    lens = w.key_lens.tolist()
    assert all(64 <= x <= 128 for x in lens)
    assert w.visible_pairs() == oracle.visible_pairs(4, 128, 128, False, w.key_lens.numpy())
    assert w.key_mask().sum().item() == sum(lens)
    full = W.config2_lens() if hasattr(W, "config2_lens") else None
    c5 = W.config5(seq=256)
    assert c5.key_lens.tolist() == [256, 256] and c5.nominal_flops() == 4.0 * 2 * 16 * 256 * 256 * 64
    w1 = W.config1()
    assert w1.q.dtype == torch.float32 and w1.scale == 0.125


def test_lens_are_the_same_for_every_layer():
    a, b = W.config2(layer=0, batch=4, seq=64), W.config2(layer=3, batch=4, seq=64)
    assert a.key_lens.tolist() == b.key_lens.tolist()
    assert not torch.equal(a.q, b.q)
