"""MI355X (gfx950) flash-attention forward and attention prologue behind the
contract of Svod's `tk` op layer.

The package is a thin host binding: ``svod_amd.ops`` mirrors
``svod_tk::ops::{attention, heads}`` (same operand layouts, option names and
error behaviour) over the C ABI of ``include/svodk.h``; the arithmetic lives in
the HIP kernels under ``csrc/``.  PyTorch is used for device memory and streams
only.
"""
from .ops import (  # noqa: F401
    Act,
    Attn,
    Cache,
    Fallback,
    GraphFallback,
    KeyMask,
    Linear,
    Rotary,
    OpError,
    Qkv,
    add_layer_norm,
    add_rms_norm,
    attention,
    attention_noalloc,
    attention_packed,
    noalloc_scratch_bytes,
    DECODE_ROWS_DEFAULT,
    tune_decode,
    tune_linear,
    tune_streaming,
    chosen,
    heads,
    layer_norm,
    linear,
    plan_linear,
    library_path,
    load_library,
    order_rows,
    plan_attention,
    plan_heads,
    plan_norm,
    rms_norm,
    supported,
)
