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

pytestmark = pytest.mark.gpu


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
                                              (64, True, 0, True)],
                         ids=["d 128, shared table", "d 64, a table row per token", "f16 without norms", "f16 without rope"])
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
