"""The code objects run as the reference's loader would run them: loaded from the file's bytes, found
by name, launched with workgroup counts and the flat argument record of device/src/hcq.rs:1262-1285
(here through the HIP runtime's module calls, which take such a record as is; the reference's own
loader writes the same record behind an AQL packet, device/src/amd/program.rs:655-760).  Results are
the library's own, bit for bit: the kernels inline the same programs."""
import ctypes
import struct

import numpy as np
import pytest
import torch

import svod_amd
from svod_amd import Attn, KeyMask, Qkv
from svod_amd import code_object as co
from util import Lcg, bf16_tensor, bits

pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("key_tiles")]  # the code objects hold the tile kernels


class Runtime:
    """hipModuleLoadData / hipModuleGetFunction / hipModuleLaunchKernel of the HIP runtime the
    process already holds."""

    def __init__(self):
        paths = sorted({line.split()[-1] for line in open("/proc/self/maps") if "libamdhip64" in line})
        assert paths, "the HIP runtime is not loaded"
        self.hip = ctypes.CDLL(paths[0])
        self.modules = {}

    def function(self, file, name):
        if file not in self.modules:
            data = (co.CO_DIR / file).read_bytes()
            module = ctypes.c_void_p()
            assert self.hip.hipModuleLoadData(ctypes.byref(module), data) == 0, file
            self.modules[file] = module
        fn = ctypes.c_void_p()
        assert self.hip.hipModuleGetFunction(ctypes.byref(fn), self.modules[file], name.encode()) == 0, name
        return fn

    def launch(self, name, values):
        """One launch of kernel `name` with the manifest's record, workgroup count and threads."""
        e = co.manifest()["kernels"][name]
        params = [tuple(p) for p in e["params"]]
        record = ctypes.create_string_buffer(co.pack(params, values, e["kernarg_size"]), e["kernarg_size"])
        size = ctypes.c_size_t(e["kernarg_size"])
        # HIP_LAUNCH_PARAM_BUFFER_POINTER, the record, HIP_LAUNCH_PARAM_BUFFER_SIZE, its size, HIP_LAUNCH_PARAM_END
        extra = (ctypes.c_void_p * 5)(1, ctypes.cast(record, ctypes.c_void_p), 2,
                                      ctypes.cast(ctypes.pointer(size), ctypes.c_void_p), 3)
        groups = eval(e["workgroups"], {k: v for k, v in values.items()})
        assert 0 < groups < 2 ** 31
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        fn = self.function(e["file"], name)
        print(f"launch {name} groups {groups} record {e['kernarg_size']} B", flush=True)
        rc = self.hip.hipModuleLaunchKernel(fn, groups, 1, 1, *e["local"], 0, stream, None, extra)
        assert rc == 0, (name, rc)
        torch.cuda.synchronize()


@pytest.fixture(scope="module")
def runtime(device):
    return Runtime()


def f32_bits(x: float) -> int:
    return struct.unpack("<i", struct.pack("<f", x))[0]


def tensor(a, device, f16):
    if f16:
        return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.float16).to(device)
    return bf16_tensor(a, device)


# (name, b, t, tk, h, hkv, d, causal, lens, f16, scale)
ATTENTION = [
    ("BGE-M3's kind: lengths, d 64", 3, 200, 200, 4, 4, 64, False, [200, 61, 0], False, None),
    ("Qwen3's kind: causal, grouped heads, d 128", 2, 300, 300, 8, 2, 128, True, [300, 130], False, None),
    ("no lengths (address 0), 11 units over 8 XCDs", 11, 130, 130, 1, 1, 64, False, None, False, None),
    ("f16, d 32, causal", 2, 100, 100, 4, 2, 32, True, None, True, None),
    ("d 48, lengths", 2, 150, 150, 4, 4, 48, False, [150, 100], False, None),
    ("f16 d 128, a scale of its own", 1, 64, 257, 2, 2, 128, False, [201], True, 0.05),
    ("cross attention, d 64 causal, queries longer than keys", 2, 260, 70, 2, 1, 64, True, None, False, None),
]


@pytest.mark.parametrize("name,b,t,tk,h,hkv,d,causal,lens,f16,scale", ATTENTION, ids=[c[0] for c in ATTENTION])
def test_attention_code_object_equals_the_library(device, runtime, name, b, t, tk, h, hkv, d, causal, lens, f16, scale):
    g = Lcg(5)
    q, k, v = (tensor(g.bf16(s), device, f16) for s in ((b, t, h, d), (b, tk, hkv, d), (b, tk, hkv, d)))
    lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=device)
    keys = KeyMask.none() if lens is None else KeyMask.lens(lens_t)
    want = svod_amd.attention(q, k, v, Attn(causal=causal, keys=keys, scale=scale, splits=1))
    assert "flash_attention" in svod_amd.chosen()
    got = torch.full_like(want, 7.0)
    kernel = f"svodk_attention_d{d}_{'f16' if f16 else 'bf16'}" + ("_causal" if causal else "")
    runtime.launch(kernel, {"q": q.data_ptr(), "k": k.data_ptr(), "v": v.data_ptr(), "o": got.data_ptr(),
                            "key_lens": 0 if lens_t is None else lens_t.data_ptr(), "batch": b, "t": t, "tk": tk,
                            "heads": h, "kv_heads": hkv, "scale_bits": f32_bits(scale if scale is not None else d ** -0.5)})
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("d,causal,f16,tk", [(64, False, False, 200), (128, True, False, 300), (64, True, True, 130),
                                             (128, False, True, 70), (64, False, False, 64 * 300)],
                         ids=["d 64", "d 128 causal", "f16 d 64 causal", "f16 d 128", "a row too long to scan up front"])
def test_key_mask_code_object_equals_the_library(device, runtime, d, causal, f16, tk):
    """The fixture of tk/src/test/unit/attention.rs:80: key j of batch row b is hidden iff (b + j) % 5 == 2;
    one row sees nothing."""
    b, t, h, hkv = 3, min(tk, 200), 4, 2
    g = Lcg(5)
    q, k, v = (tensor(g.bf16(s), device, f16) for s in ((b, t, h, d), (b, tk, hkv, d), (b, tk, hkv, d)))
    mask = np.array([[(i + j) % 5 != 2 for j in range(tk)] for i in range(b)])
    mask[1] = False
    mask_t = torch.from_numpy(mask).to(device)
    want = svod_amd.attention(q, k, v, Attn(causal=causal, keys=KeyMask.bool(mask_t), splits=1))
    assert "flash_attention" in svod_amd.chosen()
    got = torch.full_like(want, 7.0)
    kernel = f"svodk_attention_d{d}_{'f16' if f16 else 'bf16'}" + ("_causal" if causal else "") + "_mask"
    runtime.launch(kernel, {"q": q.data_ptr(), "k": k.data_ptr(), "v": v.data_ptr(), "o": got.data_ptr(),
                            "key_mask": mask_t.data_ptr(), "batch": b, "t": t, "tk": tk, "heads": h, "kv_heads": hkv,
                            "scale_bits": f32_bits(d ** -0.5)})
    assert np.array_equal(bits(got), bits(want))
    assert not bits(got[1]).any()


@pytest.mark.parametrize("d,f16,rope,norms", [(128, False, 1, True), (64, False, 2, True), (128, True, 1, False),
                                              (64, True, 0, True), (16, False, 1, True), (32, True, 2, True),
                                              (256, False, 1, True)],
                         ids=["d 128, shared table", "d 64, a table row per token", "f16 without norms", "f16 without rope",
                              "d 16", "d 32 f16, a table row per token", "d 256"])
def test_prologue_code_object_equals_the_library(device, runtime, d, f16, rope, norms):
    b, t, h, hkv = 2, 37, 4, 2
    g = Lcg(7)
    qkv = tensor(g.bf16((b, t, (h + 2 * hkv) * d), mul=3.0), device, f16)
    q_w, k_w = (tensor(g.bf16((d,), mul=0.5, add=1.0), device, f16) for _ in range(2))
    rows = b if rope == 2 else 1
    cos, sin = (tensor(g.bf16((rows, t, 1, d // 2)), device, f16) for _ in range(2))
    opts = Qkv(heads=h, kv_heads=hkv, head_dim=d, q_norm=q_w if norms else None, k_norm=k_w if norms else None, eps=1e-6,
               rope=(cos, sin) if rope else None)
    want = svod_amd.heads(qkv, opts)
    got = [torch.full_like(x, 7.0) for x in want]
    runtime.launch(f"svodk_heads_d{d}_{'f16' if f16 else 'bf16'}",
                   {"qkv": qkv.data_ptr(), "q_w": q_w.data_ptr() if norms else 0, "k_w": k_w.data_ptr() if norms else 0,
                    "cos": cos.data_ptr(), "sin": sin.data_ptr(), "q": got[0].data_ptr(), "k": got[1].data_ptr(),
                    "v": got[2].data_ptr(), "rows": b * t, "t": t, "heads": h, "kv_heads": hkv, "eps_bits": f32_bits(1e-6),
                    "rope": rope})
    for x, y in zip(got, want):
        assert np.array_equal(bits(x), bits(y))


@pytest.mark.parametrize("kind,d,f16", [("rms_norm", 1024, False), ("add_rms_norm", 2048, False), ("layer_norm", 768, False),
                                        ("add_layer_norm", 3840, True), ("add_rms_norm", 256, True), ("rms_norm", 4096, False)])
def test_norm_code_objects_equal_the_library(device, runtime, kind, d, f16):
    rows = 37  # tk/src/test/unit/rows.rs:232: a partial last block
    g = Lcg(5)
    x, r = (tensor(g.bf16((rows, d), mul=2.0, add=1.5), device, f16) for _ in range(2))
    w, b = tensor(g.bf16((d,), mul=0.5, add=1.0), device, f16), tensor(g.bf16((d,), mul=0.5), device, f16)
    eps = 1e-5
    if kind == "rms_norm":
        want = (svod_amd.rms_norm(x, w, eps),)
    elif kind == "add_rms_norm":
        want = svod_amd.add_rms_norm(x, r, w, eps)
    elif kind == "layer_norm":
        want = (svod_amd.layer_norm(x, w, b, eps),)
    else:
        want = svod_amd.add_layer_norm(x, r, w, b, eps)
    got = [torch.full_like(y, 7.0) for y in want]
    dmax = 1024 if d <= 1024 else (2048 if d <= 2048 else 4096)
    # The fused ops return (sum, y).
    values = {"x": x.data_ptr(), "residual": r.data_ptr(), "w": w.data_ptr(), "b": b.data_ptr(), "out": got[-1].data_ptr(),
              "sum": got[0].data_ptr(), "rows": rows, "d": d, "eps_bits": f32_bits(eps)}
    runtime.launch(f"svodk_{kind}_d{dmax}_{'f16' if f16 else 'bf16'}", values)
    for y, z in zip(got, want):
        assert np.array_equal(bits(y), bits(z))


# ---- the full family: every form the library has, one record for all of them.
def full_record(q, k, v, o, *, batch=None, heads=None, kv_heads=None, scale=None, key_lens=None, key_mask=None, seg_start=None,
                row_map=None, k_app=None, v_app=None, app_lens=None, bias=None, parts=None, splits=1, window=None,
                chunk=None, q_row_elems=0, kv_row_elems=0, kv_head_start=0, cache_rows=0):
    """The record of a full kernel for these operands, as the op layer would fill it
    (tk/src/ops/attention.rs:216-283: reaches capped where they no longer hide anything)."""
    ptr = lambda x: 0 if x is None else x.data_ptr()
    b, t, h, d = q.shape
    tk = k.shape[1]
    left, right = (-1, 0) if window is None else (min(window[0], t + tk), min(window[1], t + tk))
    size, cl, cr = (0, -1, 0) if chunk is None else chunk
    chunks = (t + tk) // size + 2 if size else 0
    return {"q": ptr(q), "k": ptr(k), "v": ptr(v), "o": ptr(o), "key_lens": ptr(key_lens), "key_mask": ptr(key_mask),
            "seg_start": ptr(seg_start), "row_map": ptr(row_map), "k_app": ptr(k_app), "v_app": ptr(v_app),
            "app_lens": ptr(app_lens), "bias": ptr(bias), "o_part": ptr(parts[0]) if parts else 0,
            "m_part": ptr(parts[1]) if parts else 0, "l_part": ptr(parts[2]) if parts else 0,
            "batch": batch or b, "t": t, "tk": tk, "heads": heads or h, "kv_heads": kv_heads or k.shape[2],
            "scale_bits": f32_bits(scale if scale is not None else d ** -0.5),
            "lens_i64": int(key_lens is not None and key_lens.dtype == torch.int64),
            "mask_bytes": 0 if key_mask is None else key_mask.element_size(), "q_row_elems": q_row_elems,
            "kv_row_elems": kv_row_elems, "splits": splits, "win_left": left, "win_right": right,
            "chunk_size": size, "chunk_left": -1 if cl is None else min(cl, chunks), "chunk_right": min(cr, chunks),
            "seg_i64": int(seg_start is not None and seg_start.dtype == torch.int64),
            "bias_per_batch": int(bias is not None and (bias.shape[0] != 1 or b == 1)), "kv_head_start": kv_head_start,
            "row_map_i64": int(row_map is not None and row_map.dtype == torch.int64), "cache_rows": cache_rows,
            "app_rows": 0 if k_app is None else k_app.shape[1],
            "app_lens_i64": int(app_lens is not None and app_lens.dtype == torch.int64)}


def test_full_kernels_with_per_row_ranges_equal_the_library(device, runtime):
    b, t, tk, h, hkv, d = 2, 300, 300, 4, 2, 64
    g = Lcg(5)
    q, k, v = (bf16_tensor(g.bf16(s), device) for s in ((b, t, h, d), (b, tk, hkv, d), (b, tk, hkv, d)))
    lens = torch.tensor([300, 171], dtype=torch.int32, device=device)
    seg = torch.from_numpy(np.tile(np.arange(t) - np.arange(t) % 40, (b, 1))).to(torch.int64).to(device)
    for causal, window, chunk, seg_start in ((False, (64, 64), None, None), (True, (50, 0), (32, 3, 0), seg),
                                             (False, None, (24, None, 1), None)):
        want = svod_amd.attention(q, k, v, Attn(causal=causal, keys=KeyMask.lens(lens), window=window, chunk=chunk,
                                                seg_start=seg_start, splits=1))
        got = torch.full_like(want, 7.0)
        runtime.launch(co.full_name(d, "bf16", int(causal), 0, 1, 0, 0, 0),
                       full_record(q, k, v, got, key_lens=lens, window=window, chunk=chunk, seg_start=seg_start))
        assert np.array_equal(bits(got), bits(want)), (causal, window, chunk)


def test_full_kernel_with_a_bias_and_a_key_mask_equals_the_library(device, runtime):
    b, t, tk, h, hkv, d = 2, 130, 130, 4, 2, 128
    g = Lcg(7)
    q, k, v = (tensor(g.bf16(s), device, True) for s in ((b, t, h, d), (b, tk, hkv, d), (b, tk, hkv, d)))
    bias = tensor(g.bf16((1, h, t, tk), mul=2.0), device, True)
    mask = torch.from_numpy(np.add.outer(np.arange(b), np.arange(tk)) % 5 != 2).to(device)
    want = svod_amd.attention(q, k, v, Attn(causal=True, keys=KeyMask.bool(mask), bias=bias, splits=1))
    got = torch.full_like(want, 7.0)
    runtime.launch(co.full_name(d, "f16", 1, 0, 0, 1, 0, 0), full_record(q, k, v, got, key_mask=mask, bias=bias))
    assert np.array_equal(bits(got), bits(want))


def test_full_split_kernel_and_the_merge_equal_the_library(device, runtime):
    """A decoder step: one query, 1500 keys, four splits (tk/src/test/unit/ops.rs:585), then combine_splits."""
    b, t, tk, h, d, splits = 3, 1, 1500, 20, 64, 4
    g = Lcg(9)
    q, k, v = (bf16_tensor(g.bf16(s), device) for s in ((b, t, h, d), (b, tk, h, d), (b, tk, h, d)))
    lens = torch.tensor([1500, 700, 0], dtype=torch.int32, device=device)
    want = svod_amd.attention(q, k, v, Attn(keys=KeyMask.lens(lens), splits=splits))
    assert "combine_splits" in svod_amd.chosen()
    rows = b * t * h
    parts = (torch.full((splits, rows, d), 7.0, device=device), torch.full((splits, rows), 7.0, device=device),
             torch.full((splits, rows), 7.0, device=device))
    scratch = torch.empty_like(want)
    runtime.launch(co.full_name(d, "bf16", 0, 1, 0, 0, 0, 0),
                   full_record(q, k, v, scratch, key_lens=lens, parts=parts, splits=splits))
    got = torch.full_like(want, 7.0)
    runtime.launch(f"svodk_combine_d{d}_bf16", {"o_part": parts[0].data_ptr(), "m_part": parts[1].data_ptr(),
                                                "l_part": parts[2].data_ptr(), "o": got.data_ptr(), "rows": rows,
                                                "splits": splits})
    assert np.array_equal(bits(got), bits(want))
    assert not bits(got[2]).any()


def test_full_cached_grouped_kernel_equals_the_library(device, runtime):
    """A decoder step under GQA over a cache of three layers' heads with a row map, appended rows and
    their counts (tk/src/test/unit/ops.rs:589-590), the KV head's group in one tile."""
    from svod_amd import Cache
    b, t, tk, h, hkv, d, rows, layers, appended = 5, 2, 200, 8, 2, 48, 2, 3, 8
    g = Lcg(40)
    q = bf16_tensor(g.bf16((b, t, h, d)), device)
    k, v = (bf16_tensor(g.bf16((rows, tk, layers * hkv, d)), device) for _ in range(2))
    k_app, v_app = (bf16_tensor(g.bf16((b, appended, hkv, d)), device) for _ in range(2))
    lens = torch.tensor([tk, 1, 37, tk - 1, 0], dtype=torch.int32, device=device)
    row_map = torch.tensor([0, 1, 1, 0, 1], dtype=torch.int64, device=device)
    seen = torch.tensor([8, 7, 6, 8, 1], dtype=torch.int32, device=device)
    want = svod_amd.attention(q, k, v, Attn(keys=KeyMask.lens(lens), splits=1,
                                            cache=Cache(hkv, hkv, row_map=row_map, appended=(k_app, v_app), app_lens=seen)))
    got = torch.full_like(want, 7.0)
    runtime.launch(co.full_name(d, "bf16", 0, 0, 0, 0, 1, 1),
                   full_record(q, k, v, got, kv_heads=hkv, key_lens=lens, row_map=row_map, k_app=k_app, v_app=v_app,
                               app_lens=seen, kv_row_elems=layers * hkv * d, kv_head_start=hkv, cache_rows=rows))
    assert np.array_equal(bits(got), bits(want))


def test_full_kernel_reads_a_fused_projection_in_place(device, runtime):
    """attention_packed (tk/src/ops/attention.rs:104-122): q, k and v are views of one [B, T, (H + 2 Hkv) D] row."""
    b, t, h, hkv, d = 2, 150, 4, 2, 32
    x = tensor(Lcg(3).bf16((b, t, (h + 2 * hkv) * d)), device, False)
    want = svod_amd.attention_packed(x, h, hkv, Attn(causal=True, splits=1))
    got = torch.full_like(want, 7.0)
    row = (h + 2 * hkv) * d
    q = x.view(b, t, h + 2 * hkv, d)[:, :, :h]  # shapes only: the record takes addresses
    rec = full_record(q, x.view(b, t, h + 2 * hkv, d)[:, :, h:h + hkv], None, got, heads=h, kv_heads=hkv, q_row_elems=row,
                      kv_row_elems=row)
    rec["q"], rec["k"], rec["v"] = x.data_ptr(), x.data_ptr() + h * d * 2, x.data_ptr() + (h + hkv) * d * 2
    runtime.launch(co.full_name(d, "bf16", 1, 0, 0, 0, 0, 0), rec)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("turn,f16,biased,shape", [(0, False, True, (3, 100, 96, 520)), (128, False, False, (2, 300, 256, 1024)),
                                                  (64, True, True, (2, 70, 64, 384)), (128, False, True, (17, 256, 1024, 512))],
                         ids=["plain with a bias, ragged tile edges", "24 of 32 heads of 128 turned",
                              "f16, heads of 64 turned, a bias", "17 row tiles: bands of row tiles per XCD"])
def test_linear_code_object_equals_the_library(device, runtime, turn, f16, biased, shape):
    """The projection GEMM with its rope epilogue from the code object's bytes (tk/src/kernels/gemm.rs:604-716)."""
    from svod_amd import Linear, Rotary
    b, t, k, n = shape
    g = Lcg(13)
    x = tensor(g.bf16((b, t, k)), device, f16)
    w = tensor(g.bf16((n, k), mul=0.125), device, f16)
    bias = tensor(g.bf16((n,)), device, f16) if biased else None
    heads = (n // turn) * 3 // 4 if turn else 0
    cos = sin = None
    if turn:
        cos, sin = (tensor(g.bf16((1, t, 1, turn // 2)), device, f16) for _ in range(2))
    want = svod_amd.linear(x, w, Linear(bias=bias, rope=Rotary(cos, sin, heads, turn) if turn else None))
    got = torch.full_like(want, 7.0)
    name = "svodk_linear_" + (f"rope{turn}_" if turn else "") + ("f16" if f16 else "bf16")
    runtime.launch(name, {"x": x.data_ptr(), "w": w.data_ptr(), "bias": bias.data_ptr() if biased else 0,
                          "cos": cos.data_ptr() if turn else 0, "sin": sin.data_ptr() if turn else 0, "y": got.data_ptr(),
                          "rows": b * t, "n": n, "k": k, "seq": t, "heads": heads})
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("d,h,hkv,f16", [(64, 16, 8, False), (128, 8, 8, True)], ids=["d 64, two rows a KV head", "f16 d 128"])
def test_decode_code_object_and_the_merge_equal_the_library(device, runtime, d, h, hkv, f16):
    """A decoder step over a cache of three layers' heads with a row map, appended rows and their counts, two key
    splits: the kernel that streams its keys through registers (as many workgroups as make the library launch four
    waves each, which is what the code object's kernels are fixed at), then combine_splits."""
    from svod_amd import Cache
    b, t, tk, rows, layers, appended, splits = 16, 1, 700, 3, 3, 2, 2
    g = Lcg(40)
    q = tensor(g.bf16((b, t, h, d)), device, f16)
    k, v = (tensor(g.bf16((rows, tk, layers * hkv, d)), device, f16) for _ in range(2))
    k_app, v_app = (tensor(g.bf16((b, appended, hkv, d)), device, f16) for _ in range(2))
    lens = torch.tensor([tk, 1, 37, tk - 1, 0, 64, 65, 300] * 2, dtype=torch.int32, device=device)
    row_map = torch.tensor([0, 1, 2, 0, 1, 2, 1, 0] * 2, dtype=torch.int64, device=device)
    seen = torch.tensor([2, 1, 2, 0, 1, 2, 2, 1] * 2, dtype=torch.int32, device=device)
    svod_amd.tune_decode(svod_amd.DECODE_ROWS_DEFAULT)  # this module runs key tiles otherwise
    want = svod_amd.attention(q, k, v, Attn(keys=KeyMask.lens(lens), splits=splits,
                                            cache=Cache(hkv, hkv, row_map=row_map, appended=(k_app, v_app), app_lens=seen)))
    assert "combine_splits" in svod_amd.chosen()
    n = b * t * h
    parts = (torch.full((splits, n, d), 7.0, device=device), torch.full((splits, n), 7.0, device=device),
             torch.full((splits, n), 7.0, device=device))
    kind = "f16" if f16 else "bf16"
    runtime.launch(f"svodk_decode_d{d}_r{h // hkv * t}_{kind}_s1", {
        "q": q.data_ptr(), "k": k.data_ptr(), "v": v.data_ptr(), "o": 0, "key_lens": lens.data_ptr(), "key_mask": 0,
        "row_map": row_map.data_ptr(), "k_app": k_app.data_ptr(), "v_app": v_app.data_ptr(), "app_lens": seen.data_ptr(),
        "o_part": parts[0].data_ptr(), "m_part": parts[1].data_ptr(), "l_part": parts[2].data_ptr(), "batch": b, "t": t,
        "tk": tk, "heads": h, "kv_heads": hkv, "scale_bits": f32_bits(d ** -0.5), "lens_i64": 0, "mask_bytes": 0,
        "q_row_elems": 0, "kv_row_elems": layers * hkv * d, "splits": splits, "cached": 1, "kv_head_start": hkv,
        "row_map_i64": 1, "cache_rows": rows, "app_rows": appended, "app_lens_i64": 0})
    got = torch.full_like(want, 7.0)
    runtime.launch(f"svodk_combine_d{d}_{kind}", {"o_part": parts[0].data_ptr(), "m_part": parts[1].data_ptr(),
                                                   "l_part": parts[2].data_ptr(), "o": got.data_ptr(), "rows": n,
                                                   "splits": splits})
    assert np.array_equal(bits(got), bits(want))
