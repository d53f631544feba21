"""Helpers shared by the parity tests: dtype bridges, the reference's own input
generators and its closeness rules."""
from __future__ import annotations

import numpy as np
import torch

import oracle


def to_np(t: torch.Tensor) -> np.ndarray:
    """A (bf16/f32) tensor as float32 numpy, exact."""
    return t.detach().to("cpu").to(torch.float32).numpy()


def bf16_tensor(a: np.ndarray, device) -> torch.Tensor:
    """bf16-exact float32 values as a bf16 tensor on ``device`` (the cast is exact)."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16).to(device)


def bits(t: torch.Tensor) -> np.ndarray:
    """The raw 16-bit patterns of a bf16 tensor."""
    return t.detach().to("cpu").view(torch.int16).numpy().view(np.uint16)


class Lcg:
    """``rounded(BFloat16, n, seed, f)`` of tk/src/test/unit/mod.rs:447-450 with the seed carried
    from one tensor to the next, as the reference's ``case()`` does (attention.rs:69-78)."""

    def __init__(self, seed: int):
        self.seed = seed

    def bf16(self, shape, mul=1.0, add=0.0) -> np.ndarray:
        n = int(np.prod(shape))
        out, self.seed = oracle.lcg_fill(n, self.seed, mul, add, bf16=True)
        return out.reshape(shape)


def max_abs(got: np.ndarray, want: np.ndarray) -> float:
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64)))) if got.size else 0.0


def mean_rel(got: np.ndarray, want: np.ndarray) -> float:
    """sum|got - want| / sum|want|."""
    den = float(np.sum(np.abs(want.astype(np.float64))))
    num = float(np.sum(np.abs(got.astype(np.float64) - want.astype(np.float64))))
    return num / den if den > 0 else num


def assert_rel_close(what: str, got: np.ndarray, want: np.ndarray, tol: float) -> float:
    """``|got - want| <= tol·max(|want|, 1)`` everywhere (tk/src/test/unit/mod.rs:526-536)."""
    g, w = got.astype(np.float64), want.astype(np.float64)
    diff = np.abs(g - w)
    bad = diff > tol * np.maximum(np.abs(w), 1.0)
    assert not bad.any(), f"{what}: {int(bad.sum())} elements off, worst {diff.max()} at {np.unravel_index(diff.argmax(), diff.shape)}"
    return float(diff.max()) if diff.size else 0.0


def assert_bf16_parity(what: str, got: np.ndarray, direct64: np.ndarray, program: np.ndarray,
                       max_abs_tol=2e-2, mean_rel_tol=1e-3):
    """The bar for a bf16 result.

    * max-abs <= 2e-2 against the unrounded f64 direct softmax (tk/src/test/unit/attention.rs:483);
    * mean-rel <= 1e-3 against ``program``, the reference's own tile program evaluated by the
      oracle at the kernel's tile sizes: the same algorithm, so what is left is accumulation
      order and the hardware exp2;
    * against the f64 result as a bf16 tensor stores it, no further away than that program is
      itself.  (1e-3 cannot be asked of this last comparison: the algorithm holds the
      probabilities in bf16, tk/src/kernels/attention.rs:434-435, which alone puts the
      reference's program 1.6e-3 and its graph path 2.4e-3 from the stored f64 result on the
      reference's own test inputs, and a bf16 store is 1.4e-3 from the unrounded values.)
    """
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    worst = max_abs(got, direct64)
    assert worst <= max_abs_tol, f"{what}: max-abs {worst} > {max_abs_tol}"
    mr_prog = mean_rel(got, program)
    assert mr_prog <= mean_rel_tol, f"{what}: mean-rel vs the tile program {mr_prog} > {mean_rel_tol}"
    stored = oracle.round_bf16(direct64.astype(np.float32))
    mr, mr_ref = mean_rel(got, stored), mean_rel(program, stored)
    assert mr <= max(mean_rel_tol, 1.1 * mr_ref), f"{what}: mean-rel vs f64 {mr}, the reference program's own {mr_ref}"
    return worst, mr_prog, mr
