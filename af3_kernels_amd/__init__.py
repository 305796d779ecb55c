"""MI355X-native drop-in for the attention hot path of af3_kernels.

Public names, argument order and defaults follow the reference's Python module
(src/af3_kernels/__init__.py:31-52, :108-135): `dot_product_attention_cpp`,
`pad_and_align_tensor`, `vnni_repack_tensor`, `reset_debug_timers`, `print_debug_timers`,
`print_debug_thread_imbalance`, and the two fused callers of the attention core, `_attention_cpp` (:55-80)
and `self_attention_cpp` (:83-105), with `GridSelfAttentionCpp` (src/af3_kernels/Attention.py:23-82).  Behind them a torch custom op hands raw device pointers to
libaf3_dpa.so (hand-written HIP for gfx950) through the C ABI of include/af3_dpa.h.

Inputs must live on a ROCm device; CPU tensors raise.  The attention core (`dot_product_attention_cpp`, the fp8 variant,
the casts, pad and repack helpers) runs in the HIP library or not at all: there is no CPU path and no PyTorch fallback, and
a missing library raises at first use.  The callers around the core compose it with library matrix products where a plain
GEMM is the right tool (the wide projection of the three-launch path, output projections and `Linear` layers wider than
128 columns: hipBLASLt through torch) and, for shapes outside their HIP kernels (other channel counts, float32), run the
reference module's own torch ops on the device; each function's docstring names its limits.
"""
from . import _lib
from .fused import GridSelfAttentionCpp, Linear, _attention_cpp, clear_weight_cache, gated_linear_unit_cpp, layernorm_pair_bias, self_attention_cpp  # noqa: F401
from .ops import (  # noqa: F401
    convert,
    dot_product_attention_cpp,
    dot_product_attention_fp8,
    pad_and_align_tensor,
    print_debug_thread_imbalance,
    print_debug_timers,
    quantize_fp8_e4m3,
    reset_debug_timers,
    selected_kernel,
    set_exact_bias,
    set_rows_kernel,
    vnni_repack_tensor,
)

__all__ = [
    "dot_product_attention_cpp", "dot_product_attention_fp8", "pad_and_align_tensor", "vnni_repack_tensor",
    "reset_debug_timers", "print_debug_timers", "print_debug_thread_imbalance", "convert", "quantize_fp8_e4m3",
    "selected_kernel", "set_exact_bias", "set_rows_kernel", "_attention_cpp", "self_attention_cpp", "GridSelfAttentionCpp", "layernorm_pair_bias", "gated_linear_unit_cpp", "Linear", "clear_weight_cache",
]
