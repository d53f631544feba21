"""CPU oracle for the tk flash-attention forward path and its prologue.

TEST INFRASTRUCTURE — NOT PRODUCT CODE.  Only the tests, the smoke check and
the CPU-baseline leg of the benchmark may import this package; the shipped
HIP path never does.  The arithmetic lives in ``svod_oracle.c`` (each function
cites the reference lines it restates); this module is a thin numpy/ctypes
binding plus the seeded input generators the parity tests and the benchmark
share.
"""
from __future__ import annotations

import ctypes
import dataclasses
import os
import subprocess
from dataclasses import dataclass
from typing import Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsvod_oracle.so")


def build(force: bool = False) -> str:
    """Compile ``svod_oracle.c`` with gcc (``make`` in this directory)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)
_u8p = ctypes.POINTER(ctypes.c_uint8)


class _Ranges(ctypes.Structure):
    """``svod_oracle_extras``: the chunk mask, the segment starts and the bias."""

    _fields_ = [("chunk_size", ctypes.c_int32), ("chunk_has_left", ctypes.c_int32), ("chunk_left", ctypes.c_int32),
                ("chunk_right", ctypes.c_int32), ("seg_start", ctypes.POINTER(ctypes.c_int32)),
                ("bias", ctypes.POINTER(ctypes.c_float)), ("bias_per_batch", ctypes.c_int32),
                ("bias_cols", ctypes.c_int32), ("appended", ctypes.c_int32),
                ("k_app", ctypes.POINTER(ctypes.c_float)), ("v_app", ctypes.POINTER(ctypes.c_float)),
                ("app_seen", ctypes.POINTER(ctypes.c_int32)), ("app_from", ctypes.c_int32)]


_rangesp = ctypes.POINTER(_Ranges)


def _ranges(chunk, seg_start, bias=None, batch=None, appended=None, app_from=0):
    """(pointer or None, what must stay alive) for ``chunk = (size, left or None, right)``, ``seg_start [B,T]``,
    ``bias [B or 1, H, T, Tk (+ appended rows)]`` and ``appended = (k_app, v_app, seen or None)``."""
    if chunk is None and seg_start is None and bias is None and appended is None and not app_from:
        return None, None
    r = _Ranges()
    r.app_from = int(app_from)
    seg = None
    if appended is not None:
        k_app, v_app, seen = appended
        k_app, v_app = (np.ascontiguousarray(x, dtype=np.float32) for x in (k_app, v_app))
        seen = None if seen is None else np.ascontiguousarray(seen, dtype=np.int32)
        r.appended = k_app.shape[1]
        r.k_app = k_app.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
        r.v_app = v_app.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
        if seen is not None:
            r.app_seen = seen.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
        appended = (k_app, v_app, seen)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
        r.bias = bias.ctypes.data_as(ctypes.POINTER(ctypes.c_float))
        r.bias_per_batch = int(bias.shape[0] != 1 or batch == 1)
        r.bias_cols = bias.shape[3]
    if chunk is not None:
        size, left, right = chunk
        r.chunk_size, r.chunk_has_left = int(size), int(left is not None)
        r.chunk_left, r.chunk_right = int(left or 0), int(right)
    if seg_start is not None:
        seg = np.ascontiguousarray(seg_start, dtype=np.int32)
        r.seg_start = seg.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
    return ctypes.pointer(r), (r, seg, bias, appended)

_i32 = ctypes.c_int32


def _declare(l: ctypes.CDLL) -> None:
    l.svod_oracle_round_bf16.restype = ctypes.c_double
    l.svod_oracle_round_bf16.argtypes = [ctypes.c_double]
    l.svod_oracle_round_f16.restype = ctypes.c_double
    l.svod_oracle_round_f16.argtypes = [ctypes.c_double]
    l.svod_oracle_set_stream_dtype.restype = None
    l.svod_oracle_set_stream_dtype.argtypes = [ctypes.c_int32]
    l.svod_oracle_trunc_bf16.restype = ctypes.c_double
    l.svod_oracle_trunc_bf16.argtypes = [ctypes.c_double]
    l.svod_oracle_bf16_bits.restype = ctypes.c_uint16
    l.svod_oracle_bf16_bits.argtypes = [ctypes.c_float]
    l.svod_oracle_lcg.restype = ctypes.c_double
    l.svod_oracle_lcg.argtypes = [ctypes.POINTER(ctypes.c_uint64)]
    l.svod_oracle_lcg_fill.restype = ctypes.c_uint64
    l.svod_oracle_lcg_fill.argtypes = [_f32p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_double, ctypes.c_double, ctypes.c_int]
    l.svod_oracle_normal_fill.restype = ctypes.c_uint64
    l.svod_oracle_normal_fill.argtypes = [_f32p, ctypes.c_int64, ctypes.c_uint64, ctypes.c_double, ctypes.c_int]
    l.svod_oracle_rope_table.restype = None
    l.svod_oracle_rope_table.argtypes = [ctypes.c_double, _i32, _i32, _f32p, _f32p]
    l.svod_oracle_norm_direct.restype = ctypes.c_int
    l.svod_oracle_norm_direct.argtypes = [_i32, ctypes.c_int64, _i32, ctypes.c_double, _f32p, _f32p, _f32p, _f32p, _f64p, _f32p]
    l.svod_oracle_norm_f32.restype = ctypes.c_int
    l.svod_oracle_norm_f32.argtypes = [_i32, ctypes.c_int64, _i32, ctypes.c_double, _f32p, _f32p, _f32p, _f32p, _f32p, _f32p]
    l.svod_oracle_visible.restype = None
    l.svod_oracle_visible.argtypes = [_i32, _i32, _i32, _i32, _i32, _i32, _i32p, _i32p, _i32, _rangesp, _u8p]
    l.svod_oracle_visible_pairs.restype = ctypes.c_int64
    l.svod_oracle_visible_pairs.argtypes = [_i32, _i32, _i32, _i32, _i32p]
    common = [_i32] * 6 + [_i32, _i32, _i32, ctypes.c_float, _i32p, _i32p, _i32, _rangesp]
    l.svod_oracle_attention_direct.restype = ctypes.c_int
    l.svod_oracle_attention_direct.argtypes = common + [_f32p, _f32p, _f32p, _f64p, _i32]
    l.svod_oracle_attention_graph.restype = ctypes.c_int
    l.svod_oracle_attention_graph.argtypes = common + [_i32, _f32p, _f32p, _f32p, _f32p, _i32]
    l.svod_oracle_attention_flash.restype = ctypes.c_int
    l.svod_oracle_attention_flash.argtypes = common + [_i32, _i32, _i32, _f32p, _f32p, _f32p, _f32p, _i32]
    l.svod_oracle_attention_flash_split.restype = ctypes.c_int
    l.svod_oracle_attention_flash_split.argtypes = common + [_i32, _i32, _i32, _i32, _f32p, _f32p, _f32p, _f32p, _i32]
    lin = [ctypes.c_int64, _i32, _i32, _i32, _f32p, _f32p, _f32p, _i32, _i32, _f32p, _f32p]
    l.svod_oracle_linear_direct.restype = ctypes.c_int
    l.svod_oracle_linear_direct.argtypes = lin + [_f64p]
    l.svod_oracle_linear_kernel.restype = ctypes.c_int
    l.svod_oracle_linear_kernel.argtypes = lin + [_f32p]
    heads = [_i32] * 5 + [_i32, _i32, ctypes.c_double, _i32] + [_f32p] * 5 + [_f32p] * 3
    for name in ("svod_oracle_heads_direct", "svod_oracle_heads_kernel", "svod_oracle_heads_graph"):
        getattr(l, name).restype = ctypes.c_int
        getattr(l, name).argtypes = heads


# --------------------------------------------------------------------------
# small helpers
# --------------------------------------------------------------------------
def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a: Optional[np.ndarray], ty):
    return a.ctypes.data_as(ty) if a is not None else ctypes.cast(None, ty)


def round_bf16(x):
    """tk/src/interp.rs:37-44 applied elementwise; returns float32 values that are bf16-exact."""
    a = np.ascontiguousarray(x, dtype=np.float32)
    bits = a.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
    nan = np.isnan(a)
    rounded = np.where(nan, (a.view(np.uint32) | 0x00400000) & 0xFFFF0000, rounded).astype(np.uint32)
    return rounded.view(np.float32).reshape(a.shape)


def round_f16(x):
    """The Float16 arm of tk/src/interp.rs:37-50 applied elementwise; float32 values that are f16-exact."""
    a = np.asarray(x, dtype=np.float32)
    f = np.vectorize(lambda v: lib().svod_oracle_round_f16(float(v)), otypes=[np.float64])
    return f(a).astype(np.float32)


class stream_dtype:
    """``with oracle.stream_dtype("f16"):`` — the restatements round their 16-bit values to f16
    instead of bf16 (the reference kernels run both, tk/src/ops/shape.rs:92-99)."""

    def __init__(self, name: str):
        self.which = {"bf16": 1, "f16": 2}[name]

    def __enter__(self):
        lib().svod_oracle_set_stream_dtype(self.which)
        return self

    def __exit__(self, *exc):
        lib().svod_oracle_set_stream_dtype(1)
        return False


def bf16_bits(x) -> np.ndarray:
    """The 16 stored bits of ``round_bf16(x)`` as uint16."""
    return (round_bf16(x).view(np.uint32) >> 16).astype(np.uint16)


def from_bf16_bits(bits) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def lcg_fill(n: int, seed: int, mul: float = 1.0, add: float = 0.0, bf16: bool = True):
    """``rounded(dtype, n, seed, |x| mul*x + add)`` of tk/src/test/unit/mod.rs:447-450.

    Returns ``(values float32[n], advanced_seed)``."""
    out = np.empty(n, dtype=np.float32)
    seed = lib().svod_oracle_lcg_fill(_ptr(out, _f32p), n, ctypes.c_uint64(seed), mul, add, int(bf16))
    return out, int(seed)


def normal_fill(n: int, seed: int, sigma: float = 1.0, bf16: bool = True):
    out = np.empty(n, dtype=np.float32)
    seed = lib().svod_oracle_normal_fill(_ptr(out, _f32p), n, ctypes.c_uint64(seed), sigma, int(bf16))
    return out, int(seed)


def rope_table(theta: float, seq_len: int, head_dim: int):
    """f32 ``(cos, sin)`` of shape ``[seq_len, head_dim/2]`` (tensor/src/transformer.rs:130-164)."""
    half = head_dim // 2
    cos = np.empty((seq_len, half), dtype=np.float32)
    sin = np.empty((seq_len, half), dtype=np.float32)
    lib().svod_oracle_rope_table(theta, seq_len, head_dim, _ptr(cos, _f32p), _ptr(sin, _f32p))
    return cos, sin


# --------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------
@dataclass
class Cache:
    """``Cache`` of tk/src/ops/attention.rs:39-56: k and v are ``[rows, Tk, H_all, D]`` caches."""

    head_start: int
    kv_heads: int
    row_map: Optional[np.ndarray] = None   # [B] cache row a batch lane
    appended: Optional[tuple] = None       # (k_app, v_app), each [B, n, kv_heads, D]
    app_lens: Optional[np.ndarray] = None  # [B] visible appended rows


@dataclass
class AttnProblem:
    """q [B,T,H,D]; k, v [B,Tk,Hkv,D] float32 arrays (bf16-exact when ``bf16``), or caches with ``cache``."""

    q: np.ndarray
    k: np.ndarray
    v: np.ndarray
    causal: bool = False
    key_lens: Optional[np.ndarray] = None  # [B] int
    key_mask: Optional[np.ndarray] = None  # [B, Tk] nonzero = visible
    window: Optional[tuple] = None
    chunk: Optional[tuple] = None  # (size, left or None, right): Chunk of tk/src/ops/attention.rs:39-50
    seg_start: Optional[np.ndarray] = None  # [B, T] int
    bias: Optional[np.ndarray] = None  # [B or 1, H, T, Tk] float32 (stream-dtype-exact), added to the scaled scores
    scale: Optional[float] = None
    bf16: bool = True
    cache: Optional[Cache] = None
    appended: Optional[tuple] = None  # (k_app, v_app, seen or None) beside gathered k and v: what ``gathered`` leaves
    app_from: int = 0  # the first appended column of keys that ``concatenated`` has joined (0: none): the direct softmax only

    def dims(self):
        b, t, h, d = self.q.shape
        _, tk, hkv, _ = self.k.shape
        return b, t, tk, h, hkv, d

    def gathered(self) -> "AttnProblem":
        """The cache read out as the graph reads it (tk/src/ops/attention.rs:498-503): the head range
        narrowed and the rows selected, k and v ``[B, Tk, kv_heads, D]``; appended rows kept beside them."""
        c = self.cache
        if c is None:
            return self
        rows = np.arange(self.q.shape[0]) if c.row_map is None else np.asarray(c.row_map, dtype=np.int64)
        heads = slice(c.head_start, c.head_start + c.kv_heads)
        k, v = (np.ascontiguousarray(x[rows][:, :, heads]) for x in (self.k, self.v))
        app = None
        if c.appended is not None:
            seen = None if c.app_lens is None else np.minimum(np.asarray(c.app_lens, dtype=np.int64), c.appended[0].shape[1])
            app = (c.appended[0], c.appended[1], seen)
        return dataclasses.replace(self, k=k, v=v, cache=None, appended=app)

    def concatenated(self) -> "AttnProblem":
        """Appended rows joined to the keys they follow and their visibility, with the key lengths',
        folded into one key mask (tk/src/ops/attention.rs:507-531)."""
        p = self.gathered()
        if p.appended is None:
            return p
        k_app, v_app, seen = p.appended
        b, tk, n = p.k.shape[0], p.k.shape[1], k_app.shape[1]
        lens = np.full(b, tk) if p.key_lens is None else np.minimum(np.asarray(p.key_lens, dtype=np.int64), tk)
        seen = np.full(b, n) if seen is None else seen
        mask = np.concatenate([np.arange(tk)[None, :] < lens[:, None], np.arange(n)[None, :] < seen[:, None]], axis=1)
        return dataclasses.replace(p, k=np.concatenate([p.k, k_app], axis=1), v=np.concatenate([p.v, v_app], axis=1),
                                   key_lens=None, key_mask=mask, appended=None, app_from=tk)

    def scale_f32(self) -> float:
        d = self.q.shape[-1]
        # tk/src/ops/attention.rs:230: 1.0 / (d as f32).sqrt()
        return float(self.scale) if self.scale is not None else float(np.float32(1.0) / np.sqrt(np.float32(d)))

    def _common(self):
        b, t, tk, h, hkv, d = self.dims()
        lens = None if self.key_lens is None else np.ascontiguousarray(self.key_lens, dtype=np.int32)
        mask = None if self.key_mask is None else np.ascontiguousarray(np.asarray(self.key_mask) != 0, dtype=np.int32)
        wl, wr = (-1, -1) if self.window is None else self.window
        if self.cache is not None:
            raise ValueError("a cached problem is gathered() first")
        keys = tk + (0 if self.appended is None else self.appended[0].shape[1])
        if self.bias is not None and tuple(self.bias.shape[1:]) != (h, t, keys):
            raise ValueError(f"bias has shape {self.bias.shape}, expected [{b} | 1, {h}, {t}, {keys}]")
        ranges, alive = _ranges(self.chunk, self.seg_start, self.bias, b, self.appended, self.app_from)
        keep = (lens, mask, alive)
        args = [b, t, tk, h, hkv, d, int(self.causal), wl, wr, ctypes.c_float(self.scale_f32()),
                _ptr(lens, _i32p), _ptr(mask, _i32p), tk, ranges]
        return args, keep


def attention_direct(p: AttnProblem, threads: int = 8) -> np.ndarray:
    """f64 direct softmax (tk/src/test/unit/attention.rs:102-178); unrounded float64 [B,T,H,D]."""
    p = p.concatenated()
    q, k, v = _f32(p.q), _f32(p.k), _f32(p.v)
    out = np.empty(q.shape, dtype=np.float64)
    args, _keep = p._common()
    rc = lib().svod_oracle_attention_direct(*args, _ptr(q, _f32p), _ptr(k, _f32p), _ptr(v, _f32p), _ptr(out, _f64p), threads)
    if rc:
        raise ValueError(f"oracle attention_direct rejected the problem (rc={rc})")
    return out


def attention_graph(p: AttnProblem, threads: int = 8) -> np.ndarray:
    """The op's graph fallback (tk/src/ops/attention.rs:496-584); float32 [B,T,H,D]."""
    # The graph joins the appended rows to the cached keys and masks the lot (L507-531, L573-583): unlike the
    # kernel's step for them, its causal, window, chunk and segment masks reach the appended columns too.
    p = dataclasses.replace(p.concatenated(), app_from=0)
    q, k, v = _f32(p.q), _f32(p.k), _f32(p.v)
    out = np.empty(q.shape, dtype=np.float32)
    args, _keep = p._common()
    rc = lib().svod_oracle_attention_graph(*args, int(p.bf16), _ptr(q, _f32p), _ptr(k, _f32p), _ptr(v, _f32p), _ptr(out, _f32p), threads)
    if rc:
        raise ValueError(f"oracle attention_graph rejected the problem (rc={rc})")
    return out


def attention_flash(p: AttnProblem, bq: int = 64, bkv: int = 64, threads: int = 8, splits: int = 1) -> np.ndarray:
    """The tile program under the host interpreter (tk/src/kernels/attention.rs:381-450,466-924);
    with ``splits > 1`` its keys split and the partial states merged (L609-612, L899-921, L948-1014).
    Appended rows are the last split's last step (L827-846)."""
    p = p.gathered()
    if p.appended is not None and p.appended[0].shape[1] > bkv:
        raise ValueError("the appended rows ride one key block")  # L475
    q, k, v = _f32(p.q), _f32(p.k), _f32(p.v)
    out = np.zeros(q.shape, dtype=np.float32)
    args, _keep = p._common()
    rc = lib().svod_oracle_attention_flash_split(*args, int(p.bf16), bq, bkv, int(splits), _ptr(q, _f32p), _ptr(k, _f32p), _ptr(v, _f32p), _ptr(out, _f32p), threads)
    if rc:
        raise ValueError(f"oracle attention_flash rejected the problem (rc={rc})")
    return out


def visible(batch, t, tk, causal=False, key_lens=None, key_mask=None, window=None, chunk=None, seg_start=None) -> np.ndarray:
    """uint8 [B,T,Tk]: 1 where key j is visible to query i (negated ``hidden`` of attention.rs:138-148)."""
    lens = None if key_lens is None else np.ascontiguousarray(key_lens, dtype=np.int32)
    mask = None if key_mask is None else np.ascontiguousarray(np.asarray(key_mask) != 0, dtype=np.int32)
    wl, wr = (-1, -1) if window is None else window
    out = np.empty((batch, t, tk), dtype=np.uint8)
    ranges, _alive = _ranges(chunk, seg_start)
    lib().svod_oracle_visible(batch, t, tk, int(causal), wl, wr, _ptr(lens, _i32p), _ptr(mask, _i32p), tk, ranges, _ptr(out, _u8p))
    return out


def visible_pairs(batch, t, tk, causal=False, key_lens=None) -> int:
    lens = None if key_lens is None else np.ascontiguousarray(key_lens, dtype=np.int32)
    return int(lib().svod_oracle_visible_pairs(batch, t, tk, int(causal), _ptr(lens, _i32p)))


# --------------------------------------------------------------------------
# prologue
# --------------------------------------------------------------------------
@dataclass
class HeadsProblem:
    """qkv [B,T,(H+2Hkv)*D] float32 (bf16-exact); weights [D]; tables [T,D/2] or [B,T,D/2]."""

    qkv: np.ndarray
    heads: int
    kv_heads: int
    head_dim: int
    q_w: Optional[np.ndarray] = None
    k_w: Optional[np.ndarray] = None
    eps: float = 1e-6
    cos: Optional[np.ndarray] = None
    sin: Optional[np.ndarray] = None

    def rope_kind(self) -> int:
        if self.cos is None:
            return 0
        b, t, _ = self.qkv.shape
        rows = int(np.prod(self.cos.shape)) // (self.head_dim // 2)
        if rows == t:
            return 1
        if rows == b * t:
            return 2
        raise ValueError("rope tables must hold t or batch*t rows")


def _heads(fn_name: str, p: HeadsProblem):
    b, t, width = p.qkv.shape
    h, hkv, d = p.heads, p.kv_heads, p.head_dim
    assert width == (h + 2 * hkv) * d
    qkv = _f32(p.qkv)
    q_w = None if p.q_w is None else _f32(p.q_w)
    k_w = None if p.k_w is None else _f32(p.k_w)
    cos = None if p.cos is None else _f32(p.cos)
    sin = None if p.sin is None else _f32(p.sin)
    q = np.zeros((b, t, h, d), dtype=np.float32)
    k = np.zeros((b, t, hkv, d), dtype=np.float32)
    v = np.zeros((b, t, hkv, d), dtype=np.float32)
    rc = getattr(lib(), fn_name)(b, t, h, hkv, d, int(q_w is not None), int(k_w is not None), p.eps, p.rope_kind(),
                                 _ptr(qkv, _f32p), _ptr(q_w, _f32p), _ptr(k_w, _f32p), _ptr(cos, _f32p), _ptr(sin, _f32p),
                                 _ptr(q, _f32p), _ptr(k, _f32p), _ptr(v, _f32p))
    if rc:
        raise ValueError(f"oracle {fn_name} rejected the problem (rc={rc})")
    return q, k, v


def heads_direct(p: HeadsProblem):
    """f64 reference rounded to bf16 at the store (tk/src/test/unit/heads.rs:59-105)."""
    return _heads("svod_oracle_heads_direct", p)


def heads_kernel(p: HeadsProblem):
    """heads_body under the interpreter's f32 rounding (tk/src/kernels/heads.rs:73-124)."""
    return _heads("svod_oracle_heads_kernel", p)


def heads_graph(p: HeadsProblem):
    """The op's graph fallback (tk/src/ops/heads.rs:115-134)."""
    return _heads("svod_oracle_heads_graph", p)


# --------------------------------------------------------------------------
# row norms
# --------------------------------------------------------------------------
LAYER, RMS = 0, 1


def _norm_args(x, residual, w, b):
    x = _f32(x)
    d = x.shape[-1]
    rows = x.size // d
    residual = None if residual is None else _f32(residual)
    w = _f32(w)
    b = None if b is None else _f32(b)
    if w.shape != (d,) or (b is not None and b.shape != (d,)) or (residual is not None and residual.shape != x.shape):
        raise ValueError("norm operands do not fit")
    return x, residual, w, b, rows, d


def norm_direct(kind: int, x, w, b=None, residual=None, eps: float = 1e-5):
    """The f64 reference of tk/src/test/unit/rows.rs:169-197: ``(out float64 unrounded, sum float32 or None)``."""
    x, residual, w, b, rows, d = _norm_args(x, residual, w, b)
    out = np.empty(x.shape, dtype=np.float64)
    total = None if residual is None else np.empty(x.shape, dtype=np.float32)
    rc = lib().svod_oracle_norm_direct(kind, rows, d, float(eps), _ptr(x, _f32p), _ptr(residual, _f32p), _ptr(w, _f32p),
                                       _ptr(b, _f32p), _ptr(out, _f64p), _ptr(total, _f32p))
    if rc:
        raise ValueError(f"oracle norm_direct rejected the problem (rc={rc})")
    return out, total


def norm_f32(kind: int, x, w, b=None, residual=None, eps: float = 1e-5):
    """The kernel's and the graph's f32 arithmetic (tk/src/kernels/rows.rs:73-114, tk/src/ops/norm.rs:113-127),
    rounded once to the stream dtype: ``(out float32, sum float32 or None)``."""
    x, residual, w, b, rows, d = _norm_args(x, residual, w, b)
    out = np.empty(x.shape, dtype=np.float32)
    total = None if residual is None else np.empty(x.shape, dtype=np.float32)
    rc = lib().svod_oracle_norm_f32(kind, rows, d, float(eps), _ptr(x, _f32p), _ptr(residual, _f32p), _ptr(w, _f32p),
                                    _ptr(b, _f32p), _ptr(out, _f32p), _ptr(total, _f32p))
    if rc:
        raise ValueError(f"oracle norm_f32 rejected the problem (rc={rc})")
    return out, total


# --------------------------------------------------------------------------
# linear with the rope epilogue
# --------------------------------------------------------------------------
def _linear(fn_name: str, x, w, bias, rope, out_dtype, out_ptr):
    x, w = _f32(x), _f32(w)
    if x.ndim != 3 or w.ndim != 2 or w.shape[1] != x.shape[2]:
        raise ValueError("linear: x [B, T, K] and w [N, K]")
    b, t, k = x.shape
    n = w.shape[0]
    bias = None if bias is None else _f32(bias)
    heads = head_dim = 0
    cos = sin = None
    if rope is not None:
        cos, sin, heads, head_dim = rope
        cos, sin = _f32(cos).reshape(t, head_dim // 2), _f32(sin).reshape(t, head_dim // 2)
    out = np.empty((b, t, n), dtype=out_dtype)
    rc = getattr(lib(), fn_name)(b * t, t, k, n, _ptr(x, _f32p), _ptr(w, _f32p), _ptr(bias, _f32p), heads, head_dim,
                                  _ptr(cos, _f32p), _ptr(sin, _f32p), _ptr(out, out_ptr))
    if rc:
        raise ValueError(f"oracle {fn_name} rejected the problem (rc={rc})")
    return out


def linear_direct(x, w, bias=None, rope=None) -> np.ndarray:
    """``x [B,T,K] . w [N,K]^T + bias`` with the first ``heads`` heads turned, ``rope = (cos, sin, heads, head_dim)``
    with tables ``[T, head_dim/2]``: the unrounded f64 reference of tk/src/test/unit/ops.rs:148-158."""
    return _linear("svod_oracle_linear_direct", x, w, bias, rope, np.float64, _f64p)


def linear_kernel(x, w, bias=None, rope=None) -> np.ndarray:
    """The same in the kernel's f32 arithmetic (tk/src/kernels/gemm.rs:604-716), rounded once to the stream dtype."""
    return _linear("svod_oracle_linear_kernel", x, w, bias, rope, np.float32, _f32p)
