"""Seeded synthetic inputs of the five benchmark configurations.

Every tensor is drawn from the 64-bit LCG the reference's own tests use
(``tk/src/test/unit/mod.rs:442-445``: ``seed = seed·6364136223846793005 +
1442695040888963407; u = (seed >> 33) / 2^31 · 2 − 1``), evaluated here in
closed form so it vectorises (on the GPU too); normals are Box-Muller over pairs of
draws.  Seeds: ``0x5EED0000 + 16·config + tensor_index``, plus ``1000·layer``
for the per-layer sets of config 2.  The parity tests and the benchmark share
these generators, so "the same seeded inputs" means the same bits.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np
import torch

_A = np.uint64(6364136223846793005)
_C = np.uint64(1442695040888963407)
_CHUNK = 1 << 20


def _lcg_powers(n: int):
    """a^1..a^n and 1 + a + ... + a^(k-1) for k = 1..n, modulo 2^64."""
    a = np.full(n, _A, dtype=np.uint64)
    with np.errstate(over="ignore"):
        pw = np.multiply.accumulate(a)  # a^(k+1)
        geo = np.empty(n, dtype=np.uint64)
        geo[0] = 1
        if n > 1:
            geo[1:] = np.add.accumulate(pw[:-1]) + np.uint64(1)  # 1 + a + ... + a^k
    return pw, geo


_TABLES: Dict[str, tuple] = {}


def _tables(device) -> tuple:
    """The jump tables of one chunk as int64 tensors on ``device`` (same bits as uint64)."""
    key = str(device)
    if key not in _TABLES:
        pw, geo = _lcg_powers(_CHUNK)
        with np.errstate(over="ignore"):
            cg = _C * geo
        _TABLES[key] = (torch.from_numpy(pw.view(np.int64)).to(device), torch.from_numpy(cg.view(np.int64)).to(device),
                        int(pw[-1]), int(cg[-1]))
    return _TABLES[key]


def _signed(x: int) -> int:
    x &= 0xFFFFFFFFFFFFFFFF
    return x - (1 << 64) if x >= (1 << 63) else x


def lcg_uniform(n: int, seed: int, device="cpu") -> torch.Tensor:
    """``n`` draws of the reference LCG on ``[-1, 1)`` as float64 on ``device``.

    State k of a chunk starting at ``s`` is ``a^k·s + c·(1 + a + ... + a^(k-1))``
    modulo 2^64; int64 products wrap exactly like the u64 ones."""
    pw, cg, a_m, c_m = _tables(device)
    chunks = (n + _CHUNK - 1) // _CHUNK
    starts, s = [], seed & 0xFFFFFFFFFFFFFFFF
    for _ in range(chunks):
        starts.append(_signed(s))
        s = (a_m * s + c_m) & 0xFFFFFFFFFFFFFFFF
    st = torch.tensor(starts, dtype=torch.int64, device=device)[:, None]
    states = (pw[None, :] * st + cg[None, :]).reshape(-1)[:n]
    top = (states >> 33) & 0x7FFFFFFF  # logical shift of the u64 state
    return top.to(torch.float64) / float(1 << 31) * 2.0 - 1.0


def to_bf16(x: torch.Tensor) -> torch.Tensor:
    """float32 values rounded to bf16 (nearest even, ``tk/src/interp.rs:37-44``), kept as float32."""
    return x.to(torch.float32).to(torch.bfloat16).to(torch.float32)


def normal(n: int, seed: int, sigma: float = 1.0, device="cpu") -> torch.Tensor:
    """``n`` N(0, sigma²) values, float64: Box-Muller over consecutive pairs of draws."""
    pairs = (n + 1) // 2
    u = lcg_uniform(2 * pairs, seed, device)
    u1 = 1.0 - (u[0::2] + 1.0) * 0.5  # (0, 1]
    u2 = (u[1::2] + 1.0) * 0.5
    r = sigma * torch.sqrt(-2.0 * torch.log(u1))
    ang = (2.0 * np.pi) * u2
    z = torch.stack((r * torch.cos(ang), r * torch.sin(ang)), dim=1).reshape(-1)
    return z[:n]


def uniform01(n: int, seed: int, device="cpu") -> torch.Tensor:
    return (lcg_uniform(n, seed, device) + 1.0) * 0.5


def rope_table(theta: float, seq_len: int, head_dim: int, device="cpu"):
    """f32 ``(cos, sin)`` ``[seq_len, head_dim/2]`` after ``Tensor::rope_table``
    (``tensor/src/transformer.rs:130-164``): ``inv_freq = theta^(-2i/d)``,
    ``angle = pos·inv_freq``, all in float32."""
    half = head_dim // 2
    expo = torch.arange(half, dtype=torch.float32, device=device) * float(np.float32(-2.0 / head_dim))
    inv_freq = torch.pow(torch.tensor(theta, dtype=torch.float32, device=device), expo)
    ang = torch.arange(seq_len, dtype=torch.float32, device=device)[:, None] * inv_freq[None, :]
    return torch.cos(ang), torch.sin(ang)


def seed_of(config: int, tensor_index: int, layer: int = 0) -> int:
    return 0x5EED0000 + 16 * config + tensor_index + 1000 * layer


@dataclass
class AttentionWorkload:
    """One attention call.  Tensors live on the device they were generated on, in
    the stream dtype (bf16, or f32 for config 1)."""

    name: str
    q: torch.Tensor  # [B, T, H, D]
    k: torch.Tensor  # [B, Tk, Hkv, D]
    v: torch.Tensor
    causal: bool = False
    key_lens: Optional[torch.Tensor] = None  # [B] int32
    scale: Optional[float] = None
    extra: dict = field(default_factory=dict)

    @property
    def dims(self):
        b, t, h, d = self.q.shape
        return b, t, self.k.shape[1], h, self.k.shape[2], d

    def key_mask(self) -> Optional[torch.Tensor]:
        """The ``KeyMask::Bool`` equivalent of ``key_lens``: ``[B, Tk]`` bool."""
        if self.key_lens is None:
            return None
        tk = self.k.shape[1]
        return torch.arange(tk, device=self.key_lens.device)[None, :] < self.key_lens[:, None]

    def nominal_flops(self) -> float:
        """``4·b·h·t·tk·d``, halved when causal: the reference's convention
        (``tk/examples/tk_bench.rs:277``)."""
        b, t, tk, h, _, d = self.dims
        f = 4.0 * b * h * t * tk * d
        return f / 2 if self.causal else f

    def visible_pairs(self) -> int:
        b, t, tk, _, _, _ = self.dims
        lens = [tk] * b if self.key_lens is None else [int(min(max(x, 0), tk)) for x in self.key_lens.tolist()]
        if not self.causal:
            return sum(t * n for n in lens)
        i = np.arange(t)
        return int(sum(np.minimum(i + 1, n).sum() for n in lens))

    def visible_flops(self) -> float:
        """``4·d·h·(visible (query, key) pairs)``."""
        _, _, _, h, _, d = self.dims
        return 4.0 * d * h * self.visible_pairs()

    def min_bytes(self) -> int:
        """Q + K + V + O each touched once."""
        size = self.q.element_size()
        return (2 * self.q.numel() + self.k.numel() + self.v.numel()) * size


def _tensor(shape, seed, sigma, device, dtype=torch.bfloat16):
    n = int(np.prod(shape))
    return normal(n, seed, sigma, device).to(torch.float32).to(dtype).reshape(shape)


def config1(device="cpu") -> AttentionWorkload:
    """fp32 plumbing check: B1 H1 S128 d64, N(0,1), scale 1/8, no mask."""
    shape = (1, 128, 1, 64)
    q, k, v = (_tensor(shape, seed_of(1, i), 1.0, device, torch.float32) for i in range(3))
    return AttentionWorkload("cfg1_fp32_b1_h1_s128_d64", q, k, v, scale=0.125)


def _lens(n: int, seed: int, lo: int, hi: int, device) -> torch.Tensor:
    u = uniform01(n, seed, "cpu")
    return (lo + torch.floor(u * (hi - lo + 1))).to(torch.int32).to(device)


def config2(layer: int = 0, batch: int = 32, seq: int = 512, device="cpu") -> AttentionWorkload:
    """BGE-M3 / XLM-R-large self-attention: B32 H16 d64 S512, 0.5·N(0,1), key padding U[64,512]
    (one draw per batch row, the same for every layer)."""
    shape = (batch, seq, 16, 64)
    q, k, v = (_tensor(shape, seed_of(2, i, layer), 0.5, device) for i in range(3))
    lens = _lens(batch, seed_of(2, 3), min(64, seq), seq, device)
    return AttentionWorkload(f"cfg2_bge_m3_b{batch}_h16_s{seq}_d64_layer{layer}", q, k, v, key_lens=lens, scale=0.125)


@dataclass
class PrologueWorkload:
    name: str
    qkv: torch.Tensor  # [B, T, (H + 2 Hkv) D] bf16
    q_w: torch.Tensor  # [D]
    k_w: torch.Tensor
    cos: torch.Tensor  # [1, T, 1, D/2] bf16
    sin: torch.Tensor
    heads: int
    kv_heads: int
    head_dim: int
    eps: float = 1e-6

    def min_bytes(self) -> int:
        """qkv read once, q/k/v written once, tables and weights read once."""
        return (2 * self.qkv.numel() + self.cos.numel() + self.sin.numel() + self.q_w.numel() + self.k_w.numel()) * 2


def config3_prologue(batch: int = 8, seq: int = 2048, device="cpu") -> PrologueWorkload:
    """Qwen3-Embedding-0.6B-style prologue: qkv [8,2048,(16+2·8)·128], gamma U[0.8,1.2], RoPE theta 1e6."""
    h, hkv, d = 16, 8, 128
    qkv = _tensor((batch, seq, (h + 2 * hkv) * d), seed_of(3, 0), 1.0, device)
    q_w = (0.8 + 0.4 * uniform01(d, seed_of(3, 1), device)).to(torch.float32).to(torch.bfloat16)
    k_w = (0.8 + 0.4 * uniform01(d, seed_of(3, 2), device)).to(torch.float32).to(torch.bfloat16)
    cos, sin = rope_table(1e6, seq, d, device)
    shape = (1, seq, 1, d // 2)
    return PrologueWorkload(f"cfg3_qwen3_prologue_b{batch}_s{seq}", qkv, q_w, k_w,
                            cos.to(torch.bfloat16).reshape(shape), sin.to(torch.bfloat16).reshape(shape), h, hkv, d)


def config3_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> AttentionWorkload:
    """Causal GQA attention over the prologue's outputs, right padding U[512, 2048]."""
    b, t = q.shape[0], q.shape[1]
    lens = _lens(b, seed_of(3, 3), min(512, t), t, q.device)
    return AttentionWorkload(f"cfg3_qwen3_causal_gqa_b{b}_s{t}_h16_kv8_d128", q, k, v, causal=True, key_lens=lens)


def config4(batch: int = 16, seq: int = 1500, device="cpu") -> AttentionWorkload:
    """Whisper-large-v3 encoder: B16 H20 d64 S1500, no mask, 1 % of K entries ×8."""
    shape = (batch, seq, 20, 64)
    q, k, v = (_tensor(shape, seed_of(4, i), 1.0, device) for i in range(3))
    hot = (uniform01(k.numel(), seed_of(4, 3), device) < 0.01).reshape(shape)
    k = torch.where(hot, k.to(torch.float32) * 8.0, k.to(torch.float32)).to(torch.bfloat16)
    return AttentionWorkload(f"cfg4_whisper_b{batch}_h20_s{seq}_d64", q, k, v)


def config5(seq: int = 8192, device="cpu") -> AttentionWorkload:
    """Long-context reranker pair: B2 H16 d64 S8192, lens {8192, 5000}, 0.5·N(0,1)."""
    shape = (2, seq, 16, 64)
    q, k, v = (_tensor(shape, seed_of(5, i), 0.5, device) for i in range(3))
    lens = torch.tensor([seq, min(5000, seq)], dtype=torch.int32, device=device)
    return AttentionWorkload(f"cfg5_long_b2_h16_s{seq}_d64", q, k, v, key_lens=lens)
