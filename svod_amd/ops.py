"""Host mirror of ``svod_tk::ops::{attention, heads}`` over the C ABI.

Reference: ``tk/src/ops/attention.rs:100`` (``attention``), ``tk/src/ops/heads.rs:37``
(``heads``), ``tk/src/ops/mod.rs:83-118`` (``chosen``), ``:164`` (``supported``).

The reference op "always returns a Tensor": where no kernel applies it builds
the equivalent graph itself.  That graph is Svod's, not this library's, so here
the same outcome is reported instead of computed: :class:`GraphFallback` carries
the reference's ``Fallback`` reason and the caller runs its own graph.  Nothing
in this module computes attention on the host.
"""
from __future__ import annotations

import ctypes
import enum
import os
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_NAME = "libsvodk_gfx950.so"


def library_path() -> str:
    return os.path.join(_HERE, _LIB_NAME)


class _Tensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("dtype", ctypes.c_int32), ("rank", ctypes.c_int32),
                ("shape", ctypes.c_int64 * 4)]


class _Cache(ctypes.Structure):
    _fields_ = [("head_start", ctypes.c_int64), ("kv_heads", ctypes.c_int64), ("row_map", ctypes.POINTER(_Tensor)),
                ("k_app", ctypes.POINTER(_Tensor)), ("v_app", ctypes.POINTER(_Tensor)),
                ("app_lens", ctypes.POINTER(_Tensor))]


class _Attn(ctypes.Structure):
    _fields_ = [
        ("causal", ctypes.c_int32), ("key_kind", ctypes.c_int32), ("keys", ctypes.POINTER(_Tensor)),
        ("has_window", ctypes.c_int32), ("window_left", ctypes.c_int64), ("window_right", ctypes.c_int64),
        ("has_chunk", ctypes.c_int32), ("chunk_size", ctypes.c_int64), ("chunk_has_left", ctypes.c_int32),
        ("chunk_left", ctypes.c_int64), ("chunk_right", ctypes.c_int64),
        ("seg_start", ctypes.POINTER(_Tensor)), ("cache", ctypes.POINTER(_Cache)), ("bias", ctypes.POINTER(_Tensor)),
        ("splits", ctypes.c_int32), ("has_scale", ctypes.c_int32), ("scale", ctypes.c_float),
        ("batch_live", ctypes.c_int32), ("workspace", ctypes.c_void_p), ("workspace_bytes", ctypes.c_int64),
        ("row_order", ctypes.POINTER(_Tensor)),
    ]


class _Qkv(ctypes.Structure):
    _fields_ = [
        ("heads", ctypes.c_int32), ("kv_heads", ctypes.c_int32), ("head_dim", ctypes.c_int32),
        ("q_norm", ctypes.POINTER(_Tensor)), ("k_norm", ctypes.POINTER(_Tensor)), ("eps", ctypes.c_double),
        ("cos", ctypes.POINTER(_Tensor)), ("sin", ctypes.POINTER(_Tensor)), ("batch_live", ctypes.c_int32),
    ]


class _Rotary(ctypes.Structure):
    _fields_ = [("cos", ctypes.POINTER(_Tensor)), ("sin", ctypes.POINTER(_Tensor)), ("heads", ctypes.c_int32),
                ("head_dim", ctypes.c_int32)]


class _Linear(ctypes.Structure):
    _fields_ = [("bias", ctypes.POINTER(_Tensor)), ("act", ctypes.c_int32), ("gated", ctypes.c_int32),
                ("residual", ctypes.POINTER(_Tensor)), ("has_scale", ctypes.c_int32), ("scale", ctypes.c_float),
                ("rope", ctypes.POINTER(_Rotary)), ("batch_live", ctypes.c_int32), ("has_into", ctypes.c_int32),
                ("into_at", ctypes.c_int64)]


_lib: Optional[ctypes.CDLL] = None

# Fill the outputs and workspaces this module allocates with NaN bit patterns before the call, so that
# an element a kernel leaves unwritten shows (the reference's tests do the same to their outputs,
# tk/src/test/unit/device.rs:44-50).  Off by default; the test suite turns it on.
POISON = False


def _fresh(shape, dtype, device) -> torch.Tensor:
    out = torch.empty(shape, dtype=dtype, device=device)
    if POISON and out.numel():
        if out.dtype.is_floating_point:
            out.fill_(float("nan"))
        else:
            out.view(torch.uint8).fill_(0xFF)
    return out


def load_library(path: Optional[str] = None) -> ctypes.CDLL:
    """The shared library, loaded once.  Missing library = hard error: there is
    no other implementation behind these ops.  ``path`` names another build of the same
    library and only counts on the first call."""
    global _lib
    if _lib is not None:
        return _lib
    path = path or library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m svod_amd.build` (hipcc, gfx950). "
            "svod_amd has no fallback implementation.")
    lib = ctypes.CDLL(path)
    tp = ctypes.POINTER(_Tensor)
    lib.svodk_attention.restype = ctypes.c_int
    lib.svodk_attention.argtypes = [tp, tp, tp, ctypes.POINTER(_Attn), tp, ctypes.c_void_p]
    lib.svodk_attention_noalloc.restype = ctypes.c_int
    lib.svodk_attention_noalloc.argtypes = [tp, tp, tp, ctypes.POINTER(_Attn), tp, ctypes.c_void_p]
    lib.svodk_noalloc_scratch_bytes.restype = ctypes.c_int64
    lib.svodk_attention_packed.restype = ctypes.c_int
    lib.svodk_attention_packed.argtypes = [tp, ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(_Attn), tp, ctypes.c_void_p]
    lib.svodk_attention_workspace.restype = ctypes.c_int64
    lib.svodk_attention_workspace.argtypes = [tp, tp, ctypes.POINTER(_Attn)]
    lib.svodk_heads.restype = ctypes.c_int
    lib.svodk_heads.argtypes = [tp, ctypes.POINTER(_Qkv), tp, tp, tp, ctypes.c_void_p]
    i32p, i64p = ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int64)
    lib.svodk_plan_attention.restype = ctypes.c_int
    lib.svodk_plan_attention.argtypes = [ctypes.c_int32, i32p, ctypes.c_int32, i64p, i64p, ctypes.c_int32, ctypes.c_int32]
    lib.svodk_plan_heads.restype = ctypes.c_int
    lib.svodk_plan_heads.argtypes = [ctypes.c_int32, i32p, ctypes.c_int32, i64p, ctypes.c_int32, ctypes.c_int32]
    for name, n_tensors_before_eps in (("svodk_layer_norm", 3), ("svodk_add_layer_norm", 4), ("svodk_rms_norm", 2),
                                       ("svodk_add_rms_norm", 3)):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        n_outputs = 2 if "add_" in name else 1
        fn.argtypes = [tp] * n_tensors_before_eps + [ctypes.c_double, ctypes.c_int32] + [tp] * n_outputs + [ctypes.c_void_p]
    lib.svodk_plan_norm.restype = ctypes.c_int
    lib.svodk_plan_norm.argtypes = [ctypes.c_int32, i32p, ctypes.c_int32, i64p, ctypes.c_int32]
    lib.svodk_linear.restype = ctypes.c_int
    lib.svodk_linear.argtypes = [tp, tp, ctypes.POINTER(_Linear), tp, ctypes.c_void_p]
    lib.svodk_plan_linear.restype = ctypes.c_int
    lib.svodk_plan_linear.argtypes = [ctypes.c_int32, i32p, ctypes.c_int32, i64p, ctypes.c_int32, ctypes.c_int64]
    lib.svodk_order_rows.restype = ctypes.c_int
    lib.svodk_order_rows.argtypes = [tp, tp, ctypes.c_void_p]
    lib.svodk_streaming_next_set.restype = ctypes.c_uint32
    lib.svodk_streaming_next_set.argtypes = []
    lib.svodk_tune_streaming.restype = None
    lib.svodk_tune_streaming.argtypes = [ctypes.c_int32]
    lib.svodk_tune_decode.restype = None
    lib.svodk_tune_decode.argtypes = [ctypes.c_int32]
    lib.svodk_tune_linear.restype = None
    lib.svodk_tune_linear.argtypes = [ctypes.c_int32]
    lib.svodk_supported.restype = ctypes.c_int
    lib.svodk_last_chosen.restype = ctypes.c_char_p
    lib.svodk_last_error.restype = ctypes.c_char_p
    lib.svodk_status_name.restype = ctypes.c_char_p
    lib.svodk_status_name.argtypes = [ctypes.c_int]
    lib.svodk_abi_version.restype = ctypes.c_int
    _lib = lib
    return lib


class Fallback(enum.IntEnum):
    """``Fallback`` of tk/src/ops/shape.rs:26-39."""

    Target = 1
    Dtype = 2
    Symbolic = 3
    Shape = 4
    Config = 5


class GraphFallback(Exception):
    """The op's ``Plan::Graph(why)`` outcome: no kernel applies, the caller's graph runs."""

    def __init__(self, op: str, why: Fallback):
        super().__init__(f"{op}: no kernel applies ({why.name}); run the graph op")
        self.op, self.why = op, why


class OpError(Exception):
    """``ops::Error`` of tk/src/ops/mod.rs:132-157; ``kind`` is the variant's name."""

    def __init__(self, kind: str, message: str):
        super().__init__(message)
        self.kind = kind


_ERR_KIND = {-1: "Shape", -2: "Dtype", -3: "Heads", -4: "Launch", -5: "Argument"}

_DTYPES = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2, torch.int32: 3, torch.int64: 4, torch.bool: 5}


def _desc(t: torch.Tensor) -> _Tensor:
    if t.dtype not in _DTYPES:
        raise OpError("Dtype", f"unsupported element type {t.dtype}")
    if t.dim() > 4:
        raise OpError("Shape", f"rank {t.dim()} tensor")
    if not t.is_contiguous():
        raise OpError("Argument", "operands must be dense row-major (call .contiguous())")
    d = _Tensor()
    d.data = t.data_ptr()
    d.dtype = _DTYPES[t.dtype]
    d.rank = t.dim()
    for i, s in enumerate(t.shape):
        d.shape[i] = s
    return d


def _ref(keep: list, t: Optional[torch.Tensor]):
    if t is None:
        return ctypes.POINTER(_Tensor)()
    d = _desc(t)
    keep.append(d)
    return ctypes.pointer(d)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream if t.is_cuda else 0


def _finish(op: str, status: int):
    if status == 0:
        return
    if status > 0:
        raise GraphFallback(op, Fallback(status))
    raise OpError(_ERR_KIND.get(status, "?"), load_library().svodk_last_error().decode())


@dataclass(frozen=True)
class KeyMask:
    """``KeyMask`` of tk/src/ops/attention.rs:29-37."""

    kind: int = 0
    tensor: Optional[torch.Tensor] = None

    @staticmethod
    def none() -> "KeyMask":
        return KeyMask(0, None)

    @staticmethod
    def lens(lens: torch.Tensor) -> "KeyMask":
        """``[B]`` integer valid-key counts: keys at and past ``lens[b]`` are masked."""
        return KeyMask(1, lens)

    @staticmethod
    def bool(mask: torch.Tensor) -> "KeyMask":
        """``[B, Tk]`` bool (or int32) mask, true (nonzero) where the key is attended."""
        return KeyMask(2, mask)


@dataclass
class Cache:
    """``Cache`` of tk/src/ops/attention.rs:39-56: k and v are caches ``[rows, Tk, H_all, D]``."""

    head_start: int
    kv_heads: int
    row_map: Optional[torch.Tensor] = None
    appended: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
    app_lens: Optional[torch.Tensor] = None


@dataclass
class Attn:
    """``Attn`` of tk/src/ops/attention.rs:60-86.  ``batch_live`` stands for a bound
    batch variable (``Batch::Var``): only the first ``batch_live`` batches run."""

    causal: bool = False
    keys: KeyMask = KeyMask()
    window: Optional[Tuple[int, int]] = None
    chunk: Optional[Tuple[int, Optional[int], int]] = None  # (size, left, right)
    seg_start: Optional[torch.Tensor] = None
    cache: Optional["Cache"] = None
    splits: Optional[int] = None
    scale: Optional[float] = None
    bias: Optional[torch.Tensor] = None
    batch_live: Optional[int] = None
    row_order: Optional[torch.Tensor] = None  # [B] int32 from ``order_rows``: not in the reference's Attn


@dataclass
class Qkv:
    """``Qkv`` of tk/src/ops/heads.rs:19-31."""

    heads: int
    kv_heads: int
    head_dim: int
    q_norm: Optional[torch.Tensor] = None
    k_norm: Optional[torch.Tensor] = None
    eps: float = 1e-6
    rope: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
    batch_live: Optional[int] = None


def _attn_options(opts: Attn, keep: list) -> _Attn:
    a = _Attn()
    a.causal = int(opts.causal)
    a.key_kind = opts.keys.kind
    a.keys = _ref(keep, opts.keys.tensor)
    if opts.window is not None:
        a.has_window, a.window_left, a.window_right = 1, opts.window[0], opts.window[1]
    if opts.chunk is not None:
        size, left, right = opts.chunk
        a.has_chunk, a.chunk_size, a.chunk_right = 1, size, right
        a.chunk_has_left, a.chunk_left = (0, 0) if left is None else (1, left)
    a.seg_start = _ref(keep, opts.seg_start)
    if opts.cache is not None:
        c = _Cache()
        c.head_start, c.kv_heads = int(opts.cache.head_start), int(opts.cache.kv_heads)
        c.row_map = _ref(keep, opts.cache.row_map)
        if opts.cache.appended is not None:
            c.k_app, c.v_app = _ref(keep, opts.cache.appended[0]), _ref(keep, opts.cache.appended[1])
        c.app_lens = _ref(keep, opts.cache.app_lens)
        keep.append(c)
        a.cache = ctypes.pointer(c)
    a.bias = _ref(keep, opts.bias)
    a.splits = opts.splits or 0
    if opts.scale is not None:
        a.has_scale, a.scale = 1, float(opts.scale)
    a.batch_live = opts.batch_live or 0
    a.row_order = _ref(keep, opts.row_order)
    return a


def _lend_workspace(lib, a: _Attn, qd: _Tensor, kd: _Tensor, device, workspace, keep: list) -> None:
    """The partial tensors of a split call, which the reference op allocates itself
    (tk/src/ops/attention.rs:285-293): here the harness does, like the output."""
    if a.splits == 1:
        return
    need = int(lib.svodk_attention_workspace(ctypes.byref(qd), ctypes.byref(kd), ctypes.byref(a)))
    if workspace is None and need > 0:
        workspace = _fresh(need, torch.uint8, device)
    if workspace is not None:
        keep.append(workspace)
        a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel() * workspace.element_size()


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, opts: Optional[Attn] = None,
              out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``softmax(q·kᵀ·scale)·v`` over ``q [B,T,H,D]`` and ``k``/``v [B,Tk,H_kv,D]``;
    returns ``[B,T,H,D]`` (tk/src/ops/attention.rs:98-103).  Enqueued on the
    current stream of ``q``'s device; returns without synchronising."""
    opts = opts or Attn()
    lib = load_library()
    if out is None:
        # The op allocates its output at capacity (tk/src/ops/mod.rs:423-429).
        out = _fresh(q.shape, q.dtype, q.device)
    keep: list = []
    a = _attn_options(opts, keep)
    qd, kd, vd, od = _desc(q), _desc(k), _desc(v), _desc(out)
    _lend_workspace(lib, a, qd, kd, q.device, workspace, keep)
    status = lib.svodk_attention(ctypes.byref(qd), ctypes.byref(kd), ctypes.byref(vd), ctypes.byref(a),
                                 ctypes.byref(od), ctypes.c_void_p(_stream(q)))
    _finish("attention", status)
    return out


def attention_noalloc(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, opts: Attn, out: torch.Tensor) -> torch.Tensor:
    """``attention`` through ``svodk_attention_noalloc``: the partial states of a split call live in
    the library's static device array (``noalloc_scratch_bytes()`` per GPU), nothing is allocated
    below this call, and the caller brings ``out``.  No counterpart in the reference."""
    lib = load_library()
    keep: list = []
    a = _attn_options(opts, keep)
    qd, kd, vd, od = _desc(q), _desc(k), _desc(v), _desc(out)
    status = lib.svodk_attention_noalloc(ctypes.byref(qd), ctypes.byref(kd), ctypes.byref(vd), ctypes.byref(a),
                                         ctypes.byref(od), ctypes.c_void_p(_stream(q)))
    _finish("attention", status)
    return out


def noalloc_scratch_bytes() -> int:
    return int(load_library().svodk_noalloc_scratch_bytes())


def tune_streaming(workgroups_per_xcd: int) -> None:
    """n > 0 = attention calls that can (head size 64, lengths or no key mask, no window, no splits)
    run as n streaming workgroups per XCD, each walking a run of query tiles; n <= 0 (the default)
    = a workgroup per tile.  Process-wide; results are bit-equal either way."""
    load_library().svodk_tune_streaming(int(workgroups_per_xcd))


DECODE_ROWS_DEFAULT = 2  # SVODK_DECODE_ROWS_DEFAULT of include/svodk.h


def tune_decode(rows: int) -> None:
    """The most query rows a KV head may serve (heads / kv_heads * T) for a call without causal or per-row masks
    or a bias to run as a decoder step, K and V streamed through registers: 0..4, DECODE_ROWS_DEFAULT unasked;
    0 = every call runs key tiles.  Process-wide; the two paths agree to the op's tolerance, not bit for bit."""
    load_library().svodk_tune_decode(int(rows))


def tune_linear(tile: int) -> None:
    """The output tile of every later ``linear`` call: 256 (8 waves) or 128 (4 waves); 0 = by the shape (128 where
    256 x 256 tiles would be fewer than half the compute units).  Process-wide; the two give the same bits."""
    load_library().svodk_tune_linear(int(tile))


def attention_packed(qkv: torch.Tensor, heads: int, kv_heads: int, opts: Optional[Attn] = None,
                     out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``attention`` over a fused projection ``qkv [B,T,(heads+2·kv_heads)·D]`` read in place;
    returns ``[B,T,heads,D]`` (tk/src/ops/attention.rs:104-122)."""
    opts = opts or Attn()
    lib = load_library()
    slots = heads + 2 * kv_heads
    if out is None and qkv.dim() == 3 and slots > 0 and qkv.shape[2] % slots == 0:
        out = _fresh((qkv.shape[0], qkv.shape[1], heads, qkv.shape[2] // slots), qkv.dtype, qkv.device)
    if out is None:
        out = torch.empty((1, 1, 1, 1), dtype=qkv.dtype, device=qkv.device)  # the op rejects the shape itself
    keep: list = []
    a = _attn_options(opts, keep)
    xd, od = _desc(qkv), _desc(out)
    if a.splits > 1 and qkv.dim() == 3:
        kd = _Tensor()  # the keys' view of the fused rows: [B, T, kv_heads, D]
        kd.data, kd.dtype, kd.rank = xd.data, xd.dtype, 4
        kd.shape[0], kd.shape[1], kd.shape[2], kd.shape[3] = qkv.shape[0], qkv.shape[1], kv_heads, out.shape[3]
        _lend_workspace(lib, a, od, kd, qkv.device, workspace, keep)
    status = lib.svodk_attention_packed(ctypes.byref(xd), heads, kv_heads, ctypes.byref(a), ctypes.byref(od),
                                        ctypes.c_void_p(_stream(qkv)))
    _finish("attention", status)
    return out


def heads(qkv: torch.Tensor, opts: Qkv, out: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None):
    """``qkv [B,T,(heads+2·kv_heads)·head_dim]`` → ``(q [B,T,heads,D], k, v [B,T,kv_heads,D])``
    (tk/src/ops/heads.rs:35-37)."""
    lib = load_library()
    if qkv.dim() == 3 and out is None:
        b, t = qkv.shape[0], qkv.shape[1]
        mk = lambda n: _fresh((b, t, n, opts.head_dim), qkv.dtype, qkv.device)
        out = (mk(opts.heads), mk(opts.kv_heads), mk(opts.kv_heads))
    elif out is None:
        # Let the library word the shape error; the outputs are never touched.
        e = torch.empty((0, 0, 0, 0), dtype=qkv.dtype, device=qkv.device)
        out = (e, e, e)
    keep: list = []
    o = _Qkv()
    o.heads, o.kv_heads, o.head_dim = opts.heads, opts.kv_heads, opts.head_dim
    o.q_norm, o.k_norm = _ref(keep, opts.q_norm), _ref(keep, opts.k_norm)
    o.eps = float(opts.eps)
    cos, sin = opts.rope if opts.rope is not None else (None, None)
    o.cos, o.sin = _ref(keep, cos), _ref(keep, sin)
    o.batch_live = opts.batch_live or 0
    xd, qd, kd, vd = _desc(qkv), _desc(out[0]), _desc(out[1]), _desc(out[2])
    status = lib.svodk_heads(ctypes.byref(xd), ctypes.byref(o), ctypes.byref(qd), ctypes.byref(kd), ctypes.byref(vd),
                             ctypes.c_void_p(_stream(qkv)))
    _finish("heads", status)
    return out


class Act(enum.IntEnum):
    """``Act`` of tk/src/ops/mod.rs."""

    NONE = 0
    Gelu = 1
    Silu = 2


@dataclass
class Rotary:
    """``Rotary`` of tk/src/ops/linear.rs:47-58: tables ``[1, T, 1, head_dim/2]``."""

    cos: torch.Tensor
    sin: torch.Tensor
    heads: int
    head_dim: int


@dataclass
class Linear:
    """``Linear`` of tk/src/ops/linear.rs:24-45.  ``into = (tensor [lead..., C], at)`` stores the result into the
    tensor's channels ``at .. at + N`` and returns the tensor."""

    bias: Optional[torch.Tensor] = None
    act: Act = Act.NONE
    gated: bool = False
    residual: Optional[torch.Tensor] = None
    scale: Optional[float] = None
    rope: Optional[Rotary] = None
    batch_live: Optional[int] = None
    into: Optional[Tuple[torch.Tensor, int]] = None


def linear(x: torch.Tensor, w: torch.Tensor, opts: Optional[Linear] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x [lead..., K] · w [N, K]ᵀ (+ bias)`` → ``[lead..., N]``, a fused projection's first heads rotated in the
    GEMM's store (tk/src/ops/linear.rs:60-63)."""
    opts = opts or Linear()
    lib = load_library()
    keep: list = []
    o = _Linear()
    if opts.into is not None:
        out, at = opts.into
        o.has_into, o.into_at = 1, int(at)
    if out is None:
        n = w.shape[0] // 2 if opts.gated else w.shape[0]
        out = _fresh((*x.shape[:-1], n), x.dtype, x.device)
    o.bias, o.residual = _ref(keep, opts.bias), _ref(keep, opts.residual)
    o.act, o.gated = int(opts.act), int(opts.gated)
    if opts.scale is not None:
        o.has_scale, o.scale = 1, float(opts.scale)
    if opts.rope is not None:
        r = _Rotary()
        r.cos, r.sin = _ref(keep, opts.rope.cos), _ref(keep, opts.rope.sin)
        r.heads, r.head_dim = int(opts.rope.heads), int(opts.rope.head_dim)
        keep.append(r)
        o.rope = ctypes.pointer(r)
    o.batch_live = opts.batch_live or 0
    xd, wd, od = _desc(x), _desc(w), _desc(out)
    status = lib.svodk_linear(ctypes.byref(xd), ctypes.byref(wd), ctypes.byref(o), ctypes.byref(od), ctypes.c_void_p(_stream(x)))
    _finish("linear", status)
    return out


def plan_linear(has_target: bool, dtypes, x_dims, n: int) -> Optional[Fallback]:
    """``shape::linear`` (tk/src/ops/shape.rs:120-139) as a pure function."""
    lib = load_library()
    dt = (ctypes.c_int32 * len(dtypes))(*[_DTYPES[d] for d in dtypes])
    xd = None if x_dims is None else (ctypes.c_int64 * len(x_dims))(*x_dims)
    return _plan(lib.svodk_plan_linear(int(has_target), dt, len(dtypes), xd, 0 if x_dims is None else len(x_dims), n))


def _norm(name: str, x, residual, w, b, eps, batch_live, out):
    lib = load_library()
    keep: list = []
    fused = residual is not None
    if out is None:
        out = ((_fresh(x.shape, x.dtype, x.device), _fresh(x.shape, x.dtype, x.device)) if fused
               else _fresh(x.shape, x.dtype, x.device))
    none = ctypes.POINTER(_Tensor)()
    args = [_ref(keep, x)]
    if fused:
        args.append(_ref(keep, residual))
    args.append(_ref(keep, w))
    if "layer" in name:
        args.append(_ref(keep, b) if b is not None else none)
    args += [ctypes.c_double(float(eps)), ctypes.c_int32(batch_live or 0)]
    args += [_ref(keep, out[0]), _ref(keep, out[1])] if fused else [_ref(keep, out)]
    status = getattr(lib, "svodk_" + name)(*args, ctypes.c_void_p(_stream(x)))
    _finish("layer_norm" if "layer" in name else "rms_norm", status)
    return out


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None, eps: float = 1e-5,
               out: Optional[torch.Tensor] = None, batch_live: Optional[int] = None) -> torch.Tensor:
    """``(x - mean)·rsqrt(var + eps)·w + b`` over the last dim of ``x`` (tk/src/ops/norm.rs:16-19)."""
    return _norm("layer_norm", x, None, w, b, eps, batch_live, out)


def add_layer_norm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None,
                   eps: float = 1e-5, out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                   batch_live: Optional[int] = None):
    """``(x + residual, layer_norm(x + residual))``, the sum rounded to the input type first
    (tk/src/ops/norm.rs:21-31); ``out`` is ``(sum, y)``."""
    return _norm("add_layer_norm", x, residual, w, b, eps, batch_live, out)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float = 1e-5, out: Optional[torch.Tensor] = None,
             batch_live: Optional[int] = None) -> torch.Tensor:
    """``x·rsqrt(mean(x²) + eps)·w`` over the last dim of ``x`` (tk/src/ops/norm.rs:33-36)."""
    return _norm("rms_norm", x, None, w, None, eps, batch_live, out)


def add_rms_norm(x: torch.Tensor, residual: torch.Tensor, w: torch.Tensor, eps: float = 1e-5,
                 out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, batch_live: Optional[int] = None):
    """``(x + residual, rms_norm(x + residual))``, the sum rounded to the input type first
    (tk/src/ops/norm.rs:38-42); ``out`` is ``(sum, y)``."""
    return _norm("add_rms_norm", x, residual, w, None, eps, batch_live, out)


def plan_norm(has_target: bool, dtypes, x_dims) -> Optional[Fallback]:
    """``shape::norm`` (tk/src/ops/shape.rs:221-231) as a pure function."""
    lib = load_library()
    dt = (ctypes.c_int32 * len(dtypes))(*[_DTYPES[d] for d in dtypes])
    xd = None if x_dims is None else (ctypes.c_int64 * len(x_dims))(*x_dims)
    return _plan(lib.svodk_plan_norm(int(has_target), dt, len(dtypes), xd, 0 if x_dims is None else len(x_dims)))


def order_rows(keys: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The batch rows in descending order of their key counts (ties by row) as int32 ``[B]``, for
    ``Attn.row_order``; ``keys`` is ``[B]`` lengths or a ``[B, Tk]`` key mask.  A variable-length batch whose
    rows run grouped by length ends on its short tiles."""
    lib = load_library()
    if out is None:
        out = _fresh(keys.shape[:1], torch.int32, keys.device)
    keep: list = []
    status = lib.svodk_order_rows(_ref(keep, keys), _ref(keep, out), ctypes.c_void_p(_stream(keys)))
    _finish("order_rows", status)
    return out


def chosen() -> str:
    """What the last op on this thread ran (tk/src/ops/mod.rs:83-108)."""
    return load_library().svodk_last_chosen().decode()


def supported() -> bool:
    """Whether the current device has kernels (tk/src/ops/mod.rs:164-166)."""
    return bool(load_library().svodk_supported())


def _plan(status: int) -> Optional[Fallback]:
    return None if status == 0 else Fallback(status)


def plan_attention(has_target: bool, dtypes, q_dims, k_dims, causal=False, bias=False) -> Optional[Fallback]:
    """``shape::attention`` (tk/src/ops/shape.rs:189-206) as a pure function: ``None``
    for ``Plan::Kernel``, else the ``Fallback``.  ``q_dims``/``k_dims`` ``None`` =
    a symbolic dim past the batch."""
    lib = load_library()
    dt = (ctypes.c_int32 * len(dtypes))(*[_DTYPES[d] for d in dtypes])
    qd = (ctypes.c_int64 * 4)(*q_dims) if q_dims is not None else None
    kd = (ctypes.c_int64 * 4)(*k_dims) if k_dims is not None else None
    return _plan(lib.svodk_plan_attention(int(has_target), dt, len(dtypes), qd, kd, int(causal), int(bias)))


def plan_heads(has_target: bool, dtypes, x_dims, head_dim: int) -> Optional[Fallback]:
    """``shape::heads`` (tk/src/ops/shape.rs:209-218) as a pure function."""
    lib = load_library()
    dt = (ctypes.c_int32 * len(dtypes))(*[_DTYPES[d] for d in dtypes])
    xd = (ctypes.c_int64 * len(x_dims))(*x_dims) if x_dims is not None else None
    return _plan(lib.svodk_plan_heads(int(has_target), dt, len(dtypes), xd, len(x_dims) if x_dims is not None else 0,
                                      head_dim))
