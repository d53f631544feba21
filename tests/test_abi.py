"""The C ABI without a GPU: the library loads, exports what include/svodk.h declares, validates
arguments as the reference op layer does and plans "kernel or graph" as its shape gates do.
No compute call is made here."""
import os
import re

import pytest
import torch

import svod_amd
from svod_amd import Attn, Fallback, GraphFallback, KeyMask, OpError, Qkv

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BF16, F16, F32, I32 = torch.bfloat16, torch.float16, torch.float32, torch.int32


def t(shape, dtype=BF16):
    return torch.zeros(shape, dtype=dtype)


def test_every_declared_symbol_is_exported():
    header = open(os.path.join(ROOT, "include", "svodk.h")).read()
    names = set(re.findall(r"\b(svodk_[a-z_]+)\s*\(", header))
    assert {"svodk_attention", "svodk_heads", "svodk_supported", "svodk_last_chosen"} <= names
    lib = svod_amd.load_library()
    for n in sorted(names):
        assert hasattr(lib, n), n
    assert lib.svodk_abi_version() == 8


def test_status_names():
    lib = svod_amd.load_library()
    assert lib.svodk_status_name(0) == b"Kernel"
    assert lib.svodk_status_name(4) == b"Fallback::Shape"
    assert lib.svodk_status_name(-3) == b"Error::Heads"


# ---- shape gates: tk/src/test/unit/ops_plan.rs:1153-1175 (every_op_falls_back_alike)
@pytest.mark.parametrize("has_target,dtypes,static_dims,why", [
    (False, [BF16, BF16], True, Fallback.Target),
    (True, [F32, F32], True, Fallback.Dtype),
    (True, [BF16, F32], True, Fallback.Dtype),
    (True, [I32, I32], True, Fallback.Dtype),
    (True, [BF16, BF16], False, Fallback.Symbolic),
], ids=["no target", "f32 keeps the graph", "mixed operand types", "integers", "symbolic past the batch"])
def test_every_op_falls_back_alike(has_target, dtypes, static_dims, why):
    q = [2, 128, 16, 64] if static_dims else None
    x = [2, 128, 1024] if static_dims else None
    assert svod_amd.plan_attention(has_target, dtypes, q, q) == why
    assert svod_amd.plan_heads(has_target, dtypes, x, 64) == why


# ---- ops_plan.rs:1241-1262 (attention_plans): d in {32, 48, 64, 128, 256} plan a kernel, d = 40 goes to the graph.
@pytest.mark.parametrize("d,want", [(32, None), (48, None), (64, None), (128, None), (256, None), (40, Fallback.Shape),
                                    (512, Fallback.Shape)])
def test_attention_plans(d, want):
    assert svod_amd.plan_attention(True, [BF16] * 3, [2, 100, 8, d], [2, 37, 2, d]) == want


def test_an_empty_dim_keeps_the_graph():
    assert svod_amd.plan_attention(True, [BF16] * 3, [0, 100, 8, 64], [0, 37, 2, 64]) == Fallback.Shape
    assert svod_amd.plan_heads(True, [BF16], [2, 0, 768], 64) == Fallback.Shape


def test_f16_plans_like_bf16():
    """tk/src/ops/shape.rs:92-99: either 16-bit float type takes the kernel, one type per call."""
    assert svod_amd.plan_attention(True, [F16] * 3, [2, 100, 8, 64], [2, 37, 2, 64]) is None
    assert svod_amd.plan_attention(True, [F16, BF16, F16], [2, 100, 8, 64], [2, 37, 2, 64]) == Fallback.Dtype
    assert svod_amd.plan_heads(True, [F16], [2, 100, 12 * 64], 64) is None


# ---- ops_plan.rs:1465-1487 (heads_plan and friends)
@pytest.mark.parametrize("d,want", [(64, None), (128, None), (16, None), (256, None), (48, Fallback.Shape),
                                    (512, Fallback.Shape), (8, Fallback.Shape)])
def test_heads_plan(d, want):
    assert svod_amd.plan_heads(True, [BF16], [2, 100, 12 * d], d) == want


def test_heads_keep_the_graph_for_a_weight_off_the_stream_dtype():
    assert svod_amd.plan_heads(True, [BF16, F16], [2, 100, 12 * 64], 64) == Fallback.Dtype


def test_heads_need_three_dims():
    assert svod_amd.plan_heads(True, [BF16], [200, 12 * 64], 64) == Fallback.Shape


# ---- argument errors: ops_plan.rs:1814-1879 and ops.rs:990-1002
def kind_of(fn):
    with pytest.raises(OpError) as e:
        fn()
    return e.value.kind, str(e.value)


def test_attention_rejects_what_the_graph_would_reject():
    q = t([2, 10, 6, 64])
    kv = t([2, 12, 4, 64])
    kind, msg = kind_of(lambda: svod_amd.attention(q, kv, kv))
    assert kind == "Heads" and "6 query heads" in msg and "4 key/value heads" in msg
    kv2 = t([2, 12, 2, 64])
    kind, msg = kind_of(lambda: svod_amd.attention(q, kv2, t([2, 11, 2, 64])))
    assert kind == "Shape" and msg.startswith("attention: v has shape")
    short = t([2, 12, 2, 32])
    kind, msg = kind_of(lambda: svod_amd.attention(q, short, short))
    assert kind == "Shape" and msg.startswith("attention: k has shape")
    kind, msg = kind_of(lambda: svod_amd.attention(q, kv2, kv2, Attn(keys=KeyMask.lens(t([2, 1], I32)))))
    assert kind == "Shape" and "key lens" in msg
    kind, msg = kind_of(lambda: svod_amd.attention(q, kv2, kv2, Attn(keys=KeyMask.bool(t([2, 10], torch.bool)))))
    assert kind == "Shape" and "key mask" in msg
    kind, msg = kind_of(lambda: svod_amd.attention(q, kv2, kv2, Attn(seg_start=t([2, 12], I32))))
    assert kind == "Shape" and "seg start" in msg
    kind, msg = kind_of(lambda: svod_amd.attention(t([2, 10, 64]), kv2, kv2))
    assert kind == "Shape" and "q has shape" in msg
    kind, msg = kind_of(lambda: svod_amd.attention(q, kv2.to(F16), kv2.to(F16)))
    assert kind == "Dtype" and "k is Float16" in msg
    for dims in ([2, 6, 10, 13], [3, 6, 10, 12], [2, 2, 10, 12], [2, 6, 12, 12]):
        kind, msg = kind_of(lambda: svod_amd.attention(q, kv2, kv2, Attn(bias=t(dims))))
        assert kind == "Shape" and "bias" in msg, dims


@pytest.mark.parametrize("lens", [[1], [3], [2, 1]], ids=["one length for two rows", "three lengths", "a matrix"])
def test_attention_rejects_key_lengths_off_the_batch(lens):
    """ops.rs:993-1002."""
    q, kv = t([2, 16, 4, 64]), t([2, 32, 4, 64])
    kind, msg = kind_of(lambda: svod_amd.attention(q, kv, kv, Attn(keys=KeyMask.lens(t(lens, I32)))))
    assert kind == "Shape" and "key lens" in msg


def test_heads_reject_what_the_graph_would_reject():
    x = t([2, 10, 8 * 64])
    kind, msg = kind_of(lambda: svod_amd.heads(x, Qkv(4, 3, 64)))
    assert kind == "Heads"
    kind, msg = kind_of(lambda: svod_amd.heads(t([2, 10, 7 * 64]), Qkv(4, 2, 64)))
    assert kind == "Shape" and "qkv has shape" in msg
    kind, msg = kind_of(lambda: svod_amd.heads(x, Qkv(4, 2, 64, q_norm=t([32]))))
    assert kind == "Shape" and "q norm" in msg
    kind, msg = kind_of(lambda: svod_amd.heads(x, Qkv(4, 2, 64, rope=(t([1, 9, 1, 32]), t([1, 9, 1, 32])))))
    assert kind == "Shape" and "cos has shape" in msg
    kind, msg = kind_of(lambda: svod_amd.heads(x, Qkv(4, 2, 64, rope=(t([1, 10, 1, 32]), t([2, 10, 1, 32])))))
    assert kind == "Shape" and "sin has shape" in msg


# ---- the three outcomes without a device: validation passes, then the gate says Target
def test_without_a_device_the_op_names_the_graph_and_records_it():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the Target fallback is the no-device outcome")
    q, kv = t([2, 16, 4, 64]), t([2, 32, 2, 64])
    with pytest.raises(GraphFallback) as e:
        svod_amd.attention(q, kv, kv, Attn(causal=True))
    assert e.value.why == Fallback.Target
    assert svod_amd.chosen() == 'Graph { op: "attention", why: Target }'
    with pytest.raises(GraphFallback) as e:
        svod_amd.heads(t([2, 10, 8 * 64]), Qkv(4, 2, 64))
    assert e.value.why == Fallback.Target
    assert svod_amd.chosen() == 'Graph { op: "heads", why: Target }'
    assert svod_amd.supported() is False


def test_a_missing_library_is_a_hard_error(monkeypatch, tmp_path):
    """There is no implementation behind the ops other than the HIP library."""
    import svod_amd.ops as ops

    monkeypatch.setattr(ops, "_lib", None)
    monkeypatch.setattr(ops, "_HERE", str(tmp_path))
    with pytest.raises(ImportError, match="no fallback"):
        ops.load_library()


# ---- attention_packed: tk/src/ops/attention.rs:107-114
def test_packed_attention_validates_its_operand():
    with pytest.raises(OpError) as e:
        svod_amd.attention_packed(t([2, 16, 100]), 4, 4)  # 100 is not a multiple of 12 slots
    assert e.value.kind == "Shape"
    with pytest.raises(OpError) as e:
        svod_amd.attention_packed(t([2, 16, 12 * 64]), 5, 2)
    assert e.value.kind == "Heads"
    with pytest.raises(OpError) as e:
        svod_amd.attention_packed(t([2, 16, 12 * 64]), 4, 4, Attn(cache=svod_amd.Cache(0, 4)))
    assert e.value.kind == "Shape"


def test_the_split_workspace_is_the_partial_tensors():
    """tk/src/ops/attention.rs:285-293: o_part [S,B,T,H,D] + m_part + l_part [S,B,T,H], f32; the count
    capped at the 64-key blocks of Tk (:405-410)."""
    lib = svod_amd.load_library()
    from svod_amd.ops import _attn_options, _desc
    q, k = t([2, 100, 8, 64]), t([2, 300, 2, 64])
    for asked, want in ((None, 0), (1, 0), (2, 2), (4, 4), (9, 5)):
        a = _attn_options(Attn(splits=asked), [])
        qd, kd = _desc(q), _desc(k)
        import ctypes
        got = lib.svodk_attention_workspace(ctypes.byref(qd), ctypes.byref(kd), ctypes.byref(a))
        assert got == want * 2 * 100 * 8 * (64 + 2) * 4


def test_with_no_count_named_few_query_tiles_over_many_keys_are_split():
    """tk/src/ops/attention.rs:76-79: `None` lets the tuner choose; here a rule does: enough splits for about
    512 workgroups, each with at least 8 key blocks, capped at 64; a decoder step of one or two rows a KV head
    (its own kernel) takes splits of at least 4 key blocks for about 1024 workgroups (one row) or 512 (two)."""
    import ctypes
    lib = svod_amd.load_library()
    from svod_amd.ops import _attn_options, _desc
    a = _attn_options(Attn(), [])
    # (batch, t, heads, tk) -> splits
    for (b, tq, h, tk), want in (((16, 1, 20, 1500), 3), ((1, 1, 32, 8192), 32), ((4, 16, 16, 2048), 4),
                                 ((1, 128, 16, 8192), 16), ((64, 1, 20, 1500), 1), ((32, 512, 16, 512), 1),
                                 ((1, 1, 1, 1 << 20), 64), ((2, 8192, 16, 8192), 1), ((1, 1, 4, 500), 2),
                                 ((8, 2, 8, 4096), 8), ((8, 3, 8, 4096), 8)):
        qd, kd = _desc(t([b, tq, h, 64])), _desc(t([b, tk, h, 64]))
        got = lib.svodk_attention_workspace(ctypes.byref(qd), ctypes.byref(kd), ctypes.byref(a))
        assert got == (0 if want == 1 else want * b * tq * h * (64 + 2) * 4), (b, tq, h, tk)


# ---- a cache: tk/src/ops/attention.rs:146-170
def test_a_cache_is_validated_as_the_reference_validates_it():
    from svod_amd import Cache
    q, cache_kv = t([2, 3, 4, 64]), t([5, 20, 12, 64])
    lens = KeyMask.lens(t([2], I32))
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(cache=Cache(4, 4))))
    assert kind == "Shape" and "k has shape" in msg                      # five rows, two lanes, no row map
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(cache=Cache(10, 4, row_map=t([2], I32)))))
    assert kind == "Shape" and ">= 14" in msg                            # heads 10..14 of 12
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(cache=Cache(0, 3, row_map=t([2], I32)))))
    assert kind == "Heads"
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(cache=Cache(0, 4, row_map=t([3], I32)))))
    assert kind == "Shape" and "row map" in msg
    app, short = t([2, 1, 4, 64]), t([2, 1, 2, 64])
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(keys=lens, cache=Cache(0, 4, t([2], I32), (app, short)))))
    assert kind == "Shape" and "appended v" in msg
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(cache=Cache(0, 4, t([2], I32), (app, app)))))
    assert kind == "Shape" and "key lens" in msg                         # appended rows need the prefix lengths
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(keys=lens, cache=Cache(0, 4, t([2], I32), app_lens=t([2], I32)))))
    assert kind == "Shape" and "appended lens" in msg                    # counts without rows
    kind, msg = kind_of(lambda: svod_amd.attention(q, cache_kv, cache_kv, Attn(keys=lens, bias=t([2, 4, 3, 20]), cache=Cache(0, 4, t([2], I32), (app, app)))))
    assert kind == "Shape" and "bias" in msg and "21" in msg             # the bias counts the appended row


# ---- norms: tk/src/ops/norm.rs:54-64 and tk/src/ops/config/norm.rs:19-24
@pytest.mark.parametrize("d,want", [(256, None), (768, None), (2048, None), (4096, None), (128, Fallback.Shape),
                                    (1000, Fallback.Shape), (8192, Fallback.Shape)])
def test_norm_plan(d, want):
    assert svod_amd.plan_norm(True, [BF16, BF16], [4, 37, d]) == want


def test_norm_plan_gates():
    assert svod_amd.plan_norm(False, [BF16, BF16], [37, 512]) == Fallback.Target
    assert svod_amd.plan_norm(True, [BF16, F16], [37, 512]) == Fallback.Dtype
    assert svod_amd.plan_norm(True, [torch.float32, torch.float32], [37, 512]) == Fallback.Dtype
    assert svod_amd.plan_norm(True, [BF16, BF16], None) == Fallback.Symbolic
    assert svod_amd.plan_norm(True, [BF16, BF16], [0, 512]) == Fallback.Shape


def test_norms_reject_what_the_graph_would_reject():
    x = t([2, 10, 512])
    kind, msg = kind_of(lambda: svod_amd.rms_norm(x, t([256])))
    assert kind == "Shape" and msg.startswith("rms_norm: w has shape")
    kind, msg = kind_of(lambda: svod_amd.layer_norm(x, t([512]), t([2, 512])))
    assert kind == "Shape" and msg.startswith("layer_norm: b has shape")
    kind, msg = kind_of(lambda: svod_amd.add_rms_norm(x, t([2, 9, 512]), t([512])))
    assert kind == "Shape" and "residual has shape" in msg
    kind, msg = kind_of(lambda: svod_amd.add_layer_norm(x, t([2, 10, 512]), t([512]), out=(t([2, 10, 512]), t([2, 10, 256]))))
    assert kind == "Shape" and "out has shape" in msg


def test_without_a_device_a_norm_names_the_graph():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the Target fallback is the no-device outcome")
    with pytest.raises(GraphFallback) as e:
        svod_amd.layer_norm(t([4, 512]), t([512]))
    assert e.value.why == Fallback.Target
    assert svod_amd.chosen() == 'Graph { op: "layer_norm", why: Target }'


def test_streaming_launches_take_the_counter_sets_in_turn():
    lib = svod_amd.load_library()
    sets = int(re.search(r"#define SVODK_STREAMING_SETS (\d+)", open(os.path.join(ROOT, "include", "svodk.h")).read()).group(1))
    taken = [lib.svodk_streaming_next_set() for _ in range(2 * sets + 1)]
    assert all(0 <= s < sets for s in taken)
    assert all((b - a) % sets == 1 for a, b in zip(taken, taken[1:]))  # one after another, round and round
    assert len(set(taken[:sets])) == sets  # a set is met again only after every other one
    assert taken[sets] == taken[0] and taken[2 * sets] == taken[0]
