"""The kernels as AMDGPU code objects for a loader outside the HIP runtime, and a reader that checks
a code object against what that loader asks.

The reference's device layer does not go through HIP: it parses an AMDGPU ELF, finds the kernel
descriptor `<name>.kd`, copies the image into device memory and launches with a flat argument record
(device/src/amd/program.rs:77-266 parse, :403-414 descriptor bits, :655-675 record size,
:743-746 launch sizes; device/src/hcq.rs:1262-1285 record layout; runtime/src/amd/compile.rs:190-231
file checks).  `python -m svod_amd.build --code-objects` writes `svod_amd/co/*.co` and
`manifest.json`; `check()` below restates the loader's conditions so that they can be tested
without the loader:

* ELF64, little endian, EM_AMDGPU, the gfx950 machine in e_flags' low byte;
* the symbol `<name>.kd` lies inside an allocated section and 64 bytes of descriptor follow it;
* only the relocation kinds the loader applies (ABS64, REL32, REL64, REL32_LO, REL32_HI);
* the descriptor asks for no dispatch packet, queue, dispatch id or flat scratch registers, and
  for wave64;
* kernarg_size covers the packed record (8 bytes an address, 4 a scalar, natural alignment);
* LDS within the device's 160 KiB, and fixed in the descriptor (the loader has no launch-time size).
"""
from __future__ import annotations

import json
import struct
from dataclasses import dataclass, field
from pathlib import Path
from typing import Dict, List, Sequence, Tuple

EM_AMDGPU = 224
EF_AMDGPU_MACH_GFX950 = 0x4F
LDS_LIMIT = 160 * 1024
SHF_ALLOC = 0x2
SHT_SYMTAB, SHT_RELA, SHT_DYNSYM, SHT_REL = 2, 4, 11, 9
LOADER_RELOCS = {3: "ABS64", 4: "REL32", 5: "REL64", 10: "REL32_LO", 11: "REL32_HI"}
# kernel_code_properties bits (the descriptor's u16 at byte 56).
PRIVATE_SEGMENT_BUFFER, DISPATCH_PTR, QUEUE_PTR, KERNARG_SEGMENT_PTR, DISPATCH_ID, FLAT_SCRATCH_INIT, \
    PRIVATE_SEGMENT_SIZE = (1 << i for i in range(7))
WAVEFRONT_SIZE32 = 1 << 10
USES_DYNAMIC_STACK = 1 << 11

CO_DIR = Path(__file__).resolve().parent / "co"

B, S = "buffer", "scalar"
_ATTENTION = [("q", B), ("k", B), ("v", B), ("o", B), ("key_lens", B),
              ("batch", S), ("t", S), ("tk", S), ("heads", S), ("kv_heads", S), ("scale_bits", S)]
_ATTENTION_MASK = [p if p[0] != "key_lens" else ("key_mask", B) for p in _ATTENTION]
_FULL = ([(n, B) for n in ("q", "k", "v", "o", "key_lens", "key_mask", "seg_start", "row_map", "k_app", "v_app", "app_lens",
                            "bias", "o_part", "m_part", "l_part")] +
         [(n, S) for n in ("batch", "t", "tk", "heads", "kv_heads", "scale_bits", "lens_i64", "mask_bytes", "q_row_elems",
                           "kv_row_elems", "splits", "win_left", "win_right", "chunk_size", "chunk_left", "chunk_right",
                           "seg_i64", "bias_per_batch", "kv_head_start", "row_map_i64", "cache_rows", "app_rows",
                           "app_lens_i64")])
_DECODE = ([(n, B) for n in ("q", "k", "v", "o", "key_lens", "key_mask", "row_map", "k_app", "v_app", "app_lens", "o_part",
                              "m_part", "l_part")] +
           [(n, S) for n in ("batch", "t", "tk", "heads", "kv_heads", "scale_bits", "lens_i64", "mask_bytes", "q_row_elems",
                             "kv_row_elems", "splits", "cached", "kv_head_start", "row_map_i64", "cache_rows", "app_rows",
                             "app_lens_i64")])
_COMBINE = [("o_part", B), ("m_part", B), ("l_part", B), ("o", B), ("rows", S), ("splits", S)]


def full_forms():
    """(causal, split, ranged, biased, cached, grouped) of every instantiation the library's own
    dispatch reaches: grouped tiles take neither a causal mask nor ranges."""
    for ranged, biased, cached in ((0, 0, 0), (0, 1, 0), (1, 0, 0), (1, 1, 0), (0, 0, 1), (0, 1, 1), (1, 0, 1), (1, 1, 1)):
        for causal in (0, 1):
            for split in (0, 1):
                yield causal, split, ranged, biased, cached, 0
        if not ranged:
            for split in (0, 1):
                yield 0, split, 0, biased, cached, 1


def full_name(d: int, dtype: str, causal, split, ranged, biased, cached, grouped) -> str:
    return f"svodk_attention_full_d{d}_{dtype}_c{causal}s{split}r{ranged}b{biased}k{cached}g{grouped}"


_HEADS = [("qkv", B), ("q_w", B), ("k_w", B), ("cos", B), ("sin", B), ("q", B), ("k", B), ("v", B),
          ("rows", S), ("t", S), ("heads", S), ("kv_heads", S), ("eps_bits", S), ("rope", S)]
_LINEAR = [("x", B), ("w", B), ("bias", B), ("cos", B), ("sin", B), ("y", B),
           ("rows", S), ("n", S), ("k", S), ("seq", S), ("heads", S)]
_TAIL = [("rows", S), ("d", S), ("eps_bits", S)]
_ROWS = {"rms_norm": [("x", B), ("w", B), ("out", B)] + _TAIL,
         "add_rms_norm": [("x", B), ("residual", B), ("w", B), ("out", B), ("sum", B)] + _TAIL,
         "layer_norm": [("x", B), ("w", B), ("b", B), ("out", B)] + _TAIL,
         "add_layer_norm": [("x", B), ("residual", B), ("w", B), ("b", B), ("out", B), ("sum", B)] + _TAIL}


def entries() -> Dict[str, dict]:
    """Every kernel of the code objects: its file, its parameters in record order, the threads of
    a workgroup, how many workgroups a launch takes (a Python expression over the scalars) and
    the config it stands for in the reference's terms."""
    out: Dict[str, dict] = {}
    for dtype in ("bf16", "f16"):
        for d in (32, 48, 64, 128, 256):
            for causal in (False, True):
                out[f"svodk_attention_d{d}_{dtype}" + ("_causal" if causal else "")] = {
                    "file": "svodk_attention.co", "source": "attention_kernel.hip", "params": _ATTENTION,
                    "local": [256, 1, 1],
                    "workgroups": "(batch * kv_heads + 7) // 8 * 8 * (heads // kv_heads) * ((t + 127) // 128)",
                    "op": "attention", "dtype": dtype, "head_dim": d, "causal": causal,
                    "cfg": f"FaCfg {{ bq: 128, bkv: 64, stages: 2, splits: 1, forms: {{ raw_max, skip_rescale }}, "
                           f"warp_rows: 32, core: mfma_f32_32x32x16_{dtype} }}"}
                if d >= 64:  # with a [batch, tk] byte mask in place of the lengths
                    plain = out[f"svodk_attention_d{d}_{dtype}" + ("_causal" if causal else "")]
                    out[f"svodk_attention_d{d}_{dtype}" + ("_causal" if causal else "") + "_mask"] = {
                        **plain, "params": _ATTENTION_MASK, "key_mask": True}
        for d in (32, 48, 64, 128, 256):
            for c, s, r, b, k, g in full_forms():
                per = ("1" if g else "(heads // kv_heads) * ((t + 127) // 128)") + (" * splits" if s else "")
                out[full_name(d, dtype, c, s, r, b, k, g)] = {
                    "file": f"svodk_attention_full_d{d}.co", "source": "attention_kernel.hip", "head": d, "params": _FULL,
                    "local": [256, 1, 1], "workgroups": f"(batch * kv_heads + 7) // 8 * 8 * {per}",
                    "op": "attention", "dtype": dtype, "head_dim": d, "causal": bool(c), "split": bool(s),
                    "ranged": bool(r), "biased": bool(b), "cached": bool(k), "grouped": bool(g), "key_mask": True,
                    "cfg": f"FaCfg {{ bq: 128, bkv: 64, stages: 2, splits: {'n' if s else 1}, forms: {{ raw_max, "
                           f"skip_rescale }}, warp_rows: 32, core: mfma_f32_32x32x16_{dtype} }}"}
            for rows in (1, 2, 4):  # the decoder step: at most `rows` query rows a KV head, keys streamed through registers
                for s in (0, 1):
                    out[f"svodk_decode_d{d}_r{rows}_{dtype}_s{s}"] = {
                        "file": "svodk_decode.co", "source": "decode_kernel.hip", "params": _DECODE, "local": [256, 1, 1],
                        "workgroups": "batch * kv_heads" + (" * splits" if s else ""), "op": "attention", "dtype": dtype,
                        "head_dim": d, "causal": False, "split": bool(s), "rows_per_kv_head": rows, "key_mask": True,
                        "cfg": f"FaCfg {{ rows: {rows}, lanes_per_key: {max(d, 64 if d == 48 else d) // 8}, splits: "
                               f"{'n' if s else 1}, core: v_dot2_f32_{dtype}, keys streamed through registers }}"}
            out[f"svodk_combine_d{d}_{dtype}"] = {
                "file": "svodk_combine.co", "source": "combine_kernel.hip", "params": _COMBINE, "local": [256, 1, 1],
                "workgroups": f"(rows * {d // 4} + 255) // 256", "op": "combine_splits", "dtype": dtype, "head_dim": d,
                "cfg": "NormCfg { br: 4 }"}
        for d in (16, 32, 64, 128, 256):
            out[f"svodk_heads_d{d}_{dtype}"] = {
                "file": "svodk_heads.co", "source": "heads_kernel.hip", "params": _HEADS, "local": [256, 1, 1],
                "workgroups": f"(rows * (heads + 2 * kv_heads) * {d // 16} + 255) // 256",
                "op": "heads", "dtype": dtype, "head_dim": d, "cfg": "NormCfg { lanes_per_head: d/16, block: 256 }"}
        for turn in (0, 64, 128):  # the projection GEMM, plain or with the first `heads` heads of `turn` columns turned
            out[f"svodk_linear_{'rope%d_' % turn if turn else ''}{dtype}"] = {
                "file": "svodk_linear.co", "source": "linear_kernel.hip", "params": _LINEAR, "local": [512, 1, 1],
                "workgroups": "(((rows + 255) // 256 + 7) // 8 * ((n + 255) // 256) if (rows + 255) // 256 >= 16 "
                              "else ((rows + 255) // 256 * ((n + 255) // 256) + 7) // 8) * 8",
                "op": "linear", "dtype": dtype, "rope_head_dim": turn,
                "cfg": f"GemmCfg {{ bm: 256, bn: 256, bk: 64, stages: 2, waves: 8, core: mfma_f32_32x32x16_{dtype}"
                       + (", epilogue: rope }" if turn else " }")}
        for kind, params in _ROWS.items():
            for dmax in (1024, 2048, 4096):
                out[f"svodk_{kind}_d{dmax}_{dtype}"] = {
                    "file": "svodk_rows.co", "source": "rows_kernel.hip", "params": params, "local": [256, 1, 1],
                    "workgroups": "(rows + 3) // 4", "op": kind, "dtype": dtype, "d_max": dmax,
                    "cfg": "NormCfg { br: 4 }"}
    return out


class CodeObjectError(ValueError):
    pass


@dataclass
class Descriptor:
    """The 64-byte kernel descriptor (amd_kernel_descriptor_t)."""
    group_segment_fixed_size: int
    private_segment_fixed_size: int
    kernarg_size: int
    kernel_code_entry_byte_offset: int
    compute_pgm_rsrc3: int
    compute_pgm_rsrc1: int
    compute_pgm_rsrc2: int
    kernel_code_properties: int
    kernarg_preload: int

    @classmethod
    def parse(cls, raw: bytes) -> "Descriptor":
        if len(raw) != 64:
            raise CodeObjectError("a kernel descriptor is 64 bytes")
        group, private, kernarg = struct.unpack_from("<III", raw, 0)
        (entry,) = struct.unpack_from("<q", raw, 16)
        rsrc3, rsrc1, rsrc2, props, preload = struct.unpack_from("<IIIHH", raw, 44)
        return cls(group, private, kernarg, entry, rsrc3, rsrc1, rsrc2, props, preload)

    @property
    def user_sgprs(self) -> int:
        return (self.compute_pgm_rsrc2 >> 1) & 0x1F


@dataclass
class Section:
    name: str
    kind: int
    flags: int
    addr: int
    offset: int
    size: int
    link: int
    info: int
    entsize: int


@dataclass
class CodeObject:
    """What the loader reads of an AMDGPU ELF: header fields, sections, symbols, relocations."""
    data: bytes
    e_type: int = 0
    e_machine: int = 0
    e_flags: int = 0
    sections: List[Section] = field(default_factory=list)
    symbols: Dict[str, Tuple[int, int, int]] = field(default_factory=dict)  # name -> (value, size, section)
    relocations: List[Tuple[int, int, int]] = field(default_factory=list)   # (section, offset, type)

    @classmethod
    def parse(cls, data: bytes) -> "CodeObject":
        if len(data) < 64 or data[:4] != b"\x7fELF":
            raise CodeObjectError("not an ELF")
        if data[4] != 2 or data[5] != 1:
            raise CodeObjectError("an AMDGPU code object is ELF64, little endian")
        e_type, e_machine = struct.unpack_from("<HH", data, 16)
        (shoff,) = struct.unpack_from("<Q", data, 40)
        (e_flags,) = struct.unpack_from("<I", data, 48)
        shentsize, shnum, shstrndx = struct.unpack_from("<HHH", data, 58)
        co = cls(data, e_type, e_machine, e_flags)
        raw = []
        for i in range(shnum):
            name, kind, flags, addr, offset, size, link, info, _align, entsize = struct.unpack_from(
                "<IIQQQQIIQQ", data, shoff + i * shentsize)
            raw.append((name, Section("", kind, flags, addr, offset, size, link, info, entsize)))
        strtab = raw[shstrndx][1] if shnum else None
        for name, s in raw:
            s.name = co._string(strtab, name) if strtab else ""
            co.sections.append(s)
        for s in co.sections:
            if s.kind in (SHT_SYMTAB, SHT_DYNSYM):
                names = co.sections[s.link]
                for at in range(s.offset, s.offset + s.size, s.entsize or 24):
                    st_name, _info, _other, shndx, value, size = struct.unpack_from("<IBBHQQ", data, at)
                    label = co._string(names, st_name)
                    if label:
                        co.symbols.setdefault(label, (value, size, shndx))
            elif s.kind in (SHT_RELA, SHT_REL):
                step = s.entsize or (24 if s.kind == SHT_RELA else 16)
                for at in range(s.offset, s.offset + s.size, step):
                    r_offset, r_info = struct.unpack_from("<QQ", data, at)
                    co.relocations.append((s.info, r_offset, r_info & 0xFFFFFFFF))
        return co

    def _string(self, table: Section, at: int) -> str:
        start = table.offset + at
        end = self.data.index(b"\0", start)
        return self.data[start:end].decode()

    def kernels(self) -> List[str]:
        return sorted(n[:-3] for n in self.symbols if n.endswith(".kd"))

    def descriptor(self, kernel: str) -> Descriptor:
        try:
            value, _size, shndx = self.symbols[kernel + ".kd"]
        except KeyError:
            raise CodeObjectError(f"kernel descriptor symbol '{kernel}.kd' not found") from None
        if not 0 < shndx < len(self.sections):
            raise CodeObjectError(f"'{kernel}.kd' lies in no section")
        s = self.sections[shndx]
        if not s.flags & SHF_ALLOC:
            raise CodeObjectError(f"'{kernel}.kd' lies in a section that is not loaded")
        # A linked object's symbol values are addresses, a relocatable's are section offsets.
        within = value - s.addr if s.addr else value
        if within < 0 or within + 64 > s.size:
            raise CodeObjectError(f"'{kernel}.kd' runs past its section")
        return Descriptor.parse(self.data[s.offset + within:s.offset + within + 64])


def packed_size(params: Sequence[Tuple[str, str]]) -> int:
    """Bytes of the argument record: an address is 8 bytes, a scalar 4, each at its natural
    alignment, in parameter order (device/src/hcq.rs:1278-1285)."""
    cursor = 0
    for _name, kind in params:
        width = 8 if kind == "buffer" else 4
        cursor = (cursor + width - 1) // width * width + width
    return cursor


def pack(params: Sequence[Tuple[str, str]], values: Dict[str, int], size: int) -> bytes:
    """The argument record for `values` (addresses and 32-bit scalars by parameter name), zero
    filled to `size` bytes as the loader does (device/src/amd/program.rs:680)."""
    record = bytearray(size)
    cursor = 0
    for name, kind in params:
        width = 8 if kind == "buffer" else 4
        cursor = (cursor + width - 1) // width * width
        struct.pack_into("<Q" if kind == "buffer" else "<I", record, cursor, values[name] & ((1 << 8 * width) - 1))
        cursor += width
    return bytes(record)


def check(data: bytes, kernel: str, params: Sequence[Tuple[str, str]]) -> Descriptor:
    """Raises CodeObjectError where the reference's loader would refuse `kernel` of this code
    object, or could not run it; returns its descriptor otherwise."""
    co = CodeObject.parse(data)
    if co.e_machine != EM_AMDGPU:
        raise CodeObjectError(f"e_machine {co.e_machine}, expected EM_AMDGPU ({EM_AMDGPU})")
    if co.e_type not in (1, 3):
        raise CodeObjectError("neither relocatable nor shared object")
    if co.e_flags & 0xFF != EF_AMDGPU_MACH_GFX950:
        raise CodeObjectError(f"e_flags {co.e_flags:#x}: not a gfx950 code object")
    loaded = {i for i, s in enumerate(co.sections) if s.flags & SHF_ALLOC and s.size}
    for section, offset, kind in co.relocations:
        if section in loaded and kind not in LOADER_RELOCS:
            raise CodeObjectError(f"relocation type {kind} at {offset:#x}: the loader applies only "
                                  f"{sorted(LOADER_RELOCS.values())}")
    kd = co.descriptor(kernel)
    props = kd.kernel_code_properties
    for bit, what in ((DISPATCH_PTR, "the dispatch packet"), (QUEUE_PTR, "the queue"), (DISPATCH_ID, "the dispatch id"),
                      (FLAT_SCRATCH_INIT, "flat scratch"), (PRIVATE_SEGMENT_SIZE, "the private segment size")):
        if props & bit:
            raise CodeObjectError(f"{kernel}: asks for {what} in registers, which the loader does not supply")
    if props & WAVEFRONT_SIZE32:
        raise CodeObjectError(f"{kernel}: a wave32 kernel")
    if props & USES_DYNAMIC_STACK:
        raise CodeObjectError(f"{kernel}: a dynamic stack")
    if not props & KERNARG_SEGMENT_PTR and params:
        raise CodeObjectError(f"{kernel}: takes parameters but no argument record address")
    if kd.kernarg_preload:
        raise CodeObjectError(f"{kernel}: preloads {kd.kernarg_preload} argument dwords, which a loader that writes "
                              "its own user registers does not do")
    need = packed_size(params)
    if kd.kernarg_size < need:
        raise CodeObjectError(f"{kernel}: kernarg_size {kd.kernarg_size} < the packed record's {need}")
    if kd.kernarg_size != need:
        raise CodeObjectError(f"{kernel}: kernarg_size {kd.kernarg_size} != {need}: hidden arguments follow the "
                              "parameters, and the loader would leave them zero")
    if kd.group_segment_fixed_size > LDS_LIMIT:
        raise CodeObjectError(f"{kernel}: {kd.group_segment_fixed_size} bytes of LDS")
    if kd.private_segment_fixed_size:
        raise CodeObjectError(f"{kernel}: {kd.private_segment_fixed_size} bytes of scratch a lane (spills)")
    # The entry is the descriptor's address plus this offset (program.rs:387), 256-byte aligned.
    entry = co.symbols[kernel + ".kd"][0] + kd.kernel_code_entry_byte_offset
    if co.e_type == 3 and (kd.kernel_code_entry_byte_offset == 0 or entry % 256):
        raise CodeObjectError(f"{kernel}: entry at {entry:#x}")
    return kd


def manifest() -> dict:
    """The table `python -m svod_amd.build --code-objects` writes beside the code objects."""
    path = CO_DIR / "manifest.json"
    if not path.exists():
        raise FileNotFoundError(f"{path}: run `python -m svod_amd.build --code-objects`")
    return json.loads(path.read_text())


if __name__ == "__main__":
    import sys
    for arg in sys.argv[1:]:
        co = CodeObject.parse(Path(arg).read_bytes())
        print(f"{arg}: e_flags {co.e_flags:#x}, {len(co.relocations)} relocations")
        for k in co.kernels():
            kd = co.descriptor(k)
            print(f"  {k}: kernarg {kd.kernarg_size} B, LDS {kd.group_segment_fixed_size} B, scratch "
                  f"{kd.private_segment_fixed_size} B, properties {kd.kernel_code_properties:#06x}, "
                  f"preload {kd.kernarg_preload}, user sgprs {kd.user_sgprs}")
