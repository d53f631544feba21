"""The kernels as code objects for the reference's own loader (device/src/amd/program.rs:77-266,
403-414, 655-675; device/src/hcq.rs:1262-1285): every kernel of every built file meets what that
loader asks, the argument record is packed as the loader packs it (the reference's own vectors,
device/src/test/unit/hcq.rs:24-46), and the checker refuses what the loader would refuse."""
import os
import struct

import pytest

from svod_amd import code_object as co


@pytest.fixture(scope="module")
def built():
    table = co.entries()
    files = {e["file"] for e in table.values()}
    if not all((co.CO_DIR / f).exists() for f in files):
        from svod_amd import build
        build.build_code_objects()
    return {f: (co.CO_DIR / f).read_bytes() for f in files}


def test_the_record_is_packed_as_the_loader_packs_it():
    # hcq.rs:24-35: two buffers, two scalars: 24 bytes, -2 and 0x12345678 as 4-byte integers.
    dense = [("a", co.B), ("b", co.B), ("low", co.S), ("high", co.S)]
    assert co.packed_size(dense) == 24
    rec = co.pack(dense, {"a": 0x1122334455667788, "b": 0x99AABBCCDDEEFF00, "low": -2, "high": 0x12345678}, 32)
    assert rec[0:8] == (0x1122334455667788).to_bytes(8, "little")
    assert rec[8:16] == (0x99AABBCCDDEEFF00).to_bytes(8, "little")
    assert rec[16:20] == struct.pack("<i", -2) and rec[20:24] == struct.pack("<i", 0x12345678)
    assert rec[24:] == bytes(8)
    # hcq.rs:37-46: a buffer after a scalar is realigned, not packed tight.
    sparse = [("a", co.B), ("n", co.S), ("b", co.B)]
    assert co.packed_size(sparse) == 24
    rec = co.pack(sparse, {"a": 0x1000, "n": 7, "b": 0x5000}, 24)
    assert rec[:8] == (0x1000).to_bytes(8, "little") and rec[8:12] == struct.pack("<i", 7)
    assert rec[12:16] == bytes(4) and rec[16:24] == (0x5000).to_bytes(8, "little")
    # hcq.rs:60-72: buffer, scalar, buffer, scalar: 28 bytes.
    assert co.packed_size([("a", co.B), ("x", co.S), ("b", co.B), ("y", co.S)]) == 28


def test_every_kernel_meets_the_loaders_conditions(built):
    table = co.entries()
    # the short records (attention 32, prologue 10, norms 24, projection 6), every form of every head size and type, the
    # merges, the decoder step (1, 2 or 4 rows a KV head, split or not)
    assert len(table) == 72 + 5 * 2 * 40 + 10 + 5 * 2 * 3 * 2
    assert len(list(co.full_forms())) == 40
    for name, e in table.items():
        kd = co.check(built[e["file"]], name, e["params"])
        assert kd.kernarg_size == co.packed_size(e["params"]), name
        assert kd.kernel_code_properties == co.KERNARG_SEGMENT_PTR, name  # the record's address and nothing else
        assert kd.user_sgprs == 2 and kd.kernarg_preload == 0, name
        assert kd.private_segment_fixed_size == 0, name
        if "rows_per_kv_head" in e:
            # The decoder step holds no keys in LDS: ten floats (m, l, eight columns) a row, a lane of a key row and a
            # wave, for the merge of up to eight waves at the end.
            wide = 64 if e["head_dim"] == 48 else e["head_dim"]
            assert kd.group_segment_fixed_size == 8 * e["rows_per_kv_head"] * (wide // 8) * 10 * 4, name
        elif e["op"] == "attention":
            # The K and V ring: two slots each of 64 keys (tk/src/kernels/attention.rs:187-190).
            # and behind it, with a key mask, a 64-bit word a key block for each of 4 waves (256 blocks scanned).
            mask_words = 4 * 256 * 8 if e.get("key_mask") else 0
            wide = 64 if e["head_dim"] == 48 else e["head_dim"]  # a head of 48 takes the 64-wide tile
            assert kd.group_segment_fixed_size == 2 * 2 * 64 * wide * 2 + mask_words, name
        elif e["op"] == "linear":
            assert kd.group_segment_fixed_size == 2 * 2 * 256 * 64 * 2, name  # two stages of a W and an X tile of 64 k-columns
        else:
            assert kd.group_segment_fixed_size == 0, name


def test_the_files_hold_the_tables_kernels_and_nothing_to_relocate(built):
    table = co.entries()
    for f, data in built.items():
        obj = co.CodeObject.parse(data)
        assert obj.e_machine == co.EM_AMDGPU and obj.e_flags & 0xFF == co.EF_AMDGPU_MACH_GFX950
        assert set(obj.kernels()) == {n for n, e in table.items() if e["file"] == f}
        loaded = {i for i, s in enumerate(obj.sections) if s.flags & co.SHF_ALLOC}
        assert all(kind in co.LOADER_RELOCS for sec, _off, kind in obj.relocations if sec in loaded)


def test_the_manifest_lists_what_a_binding_needs(built):
    m = co.manifest()
    assert m["arch"] == "gfx950" and set(m["kernels"]) == set(co.entries())
    k = m["kernels"]["svodk_attention_d128_bf16_causal"]
    assert [p[0] for p in k["params"]] == ["q", "k", "v", "o", "key_lens", "batch", "t", "tk", "heads", "kv_heads", "scale_bits"]
    assert k["kernarg_size"] == 64 and k["lds_bytes"] == 65536 and k["local"] == [256, 1, 1]
    # cfg3: B8 T2048 H16 Hkv8 -> 64 units of 2 heads x 16 tiles.
    assert eval(k["workgroups"], {"batch": 8, "t": 2048, "heads": 16, "kv_heads": 8}) == 64 * 2 * 16
    n = m["kernels"]["svodk_add_rms_norm_d2048_bf16"]
    assert eval(n["workgroups"], {"rows": 37}) == 10 and n["kernarg_size"] == 52


def patched(data: bytes, kernel: str, at: int, fmt: str, value: int) -> bytes:
    obj = co.CodeObject.parse(data)
    addr, _size, shndx = obj.symbols[kernel + ".kd"]
    s = obj.sections[shndx]
    where = s.offset + (addr - s.addr if s.addr else addr) + at
    out = bytearray(data)
    struct.pack_into(fmt, out, where, value)
    return bytes(out)


def test_the_checker_refuses_what_the_loader_would(built):
    name = "svodk_heads_d128_bf16"
    e = co.entries()[name]
    data = built[e["file"]]
    co.check(data, name, e["params"])
    with pytest.raises(co.CodeObjectError, match="not an ELF"):
        co.check(b"\0" * 128, name, e["params"])
    with pytest.raises(co.CodeObjectError, match="e_machine"):
        co.check(data[:18] + b"\x3e\x00" + data[20:], name, e["params"])  # x86-64
    with pytest.raises(co.CodeObjectError, match="gfx950"):
        co.check(data[:48] + b"\x4c" + data[49:], name, e["params"])  # gfx942's machine number
    with pytest.raises(co.CodeObjectError, match="not found"):
        co.check(data, "svodk_heads_d96_bf16", e["params"])
    # program.rs:403-414: a kernel that wants the dispatch packet's address is refused at load.
    with pytest.raises(co.CodeObjectError, match="dispatch packet"):
        co.check(patched(data, name, 56, "<H", co.KERNARG_SEGMENT_PTR | co.DISPATCH_PTR), name, e["params"])
    # program.rs:663-675: the record must fit kernarg_size.
    with pytest.raises(co.CodeObjectError, match="kernarg_size"):
        co.check(data, name, e["params"] + [("one_more", co.B)])
    with pytest.raises(co.CodeObjectError, match="hidden"):
        co.check(patched(data, name, 8, "<I", 88 + 256), name, e["params"])
    # program.rs:367-375: more LDS than the device has.
    with pytest.raises(co.CodeObjectError, match="LDS"):
        co.check(patched(data, name, 0, "<I", 161 * 1024), name, e["params"])
    with pytest.raises(co.CodeObjectError, match="preload"):
        co.check(patched(data, name, 58, "<H", 14), name, e["params"])


def test_a_missing_build_is_said_plainly(tmp_path, monkeypatch):
    monkeypatch.setattr(co, "CO_DIR", tmp_path)
    with pytest.raises(FileNotFoundError, match="code-objects"):
        co.manifest()
