"""ctypes binding of libaf3_dpa.so (the C ABI declared in include/af3_dpa.h).

There is no fallback: if the library is missing, loading raises and every op fails loudly.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libaf3_dpa.so")

AF3_F32, AF3_BF16, AF3_FP8_E4M3, AF3_FP8_E5M2 = 0, 1, 2, 3
ABI_VERSION = 4
STATIC_SCRATCH_BYTES = 16 * 1024 * 1024   # AF3_STATIC_SCRATCH_BYTES

i64, i32, f32, vp = ctypes.c_int64, ctypes.c_int32, ctypes.c_float, ctypes.c_void_p


class DpaParams(ctypes.Structure):
    """Mirror of struct af3_dpa_params."""
    _fields_ = [
        ("q", vp), ("k", vp), ("v", vp), ("bias", vp), ("key_mask", vp), ("out", vp),
        ("B", i64), ("H", i64), ("L", i64), ("D", i64),
        ("q_stride", i64 * 3), ("k_stride", i64 * 3), ("v_stride", i64 * 3), ("out_stride", i64 * 3),
        ("bias_stride", i64 * 2), ("key_mask_stride_b", i64),
        ("io_dtype", i32), ("bias_dtype", i32), ("out_dtype", i32), ("mma_dtype", i32),
        ("softmax_scale", f32), ("q_descale", f32), ("k_descale", f32), ("v_descale", f32),
        ("force_generic", i32), ("reserved", i32),
        ("device_descales", vp),
        ("workspace", vp), ("workspace_bytes", i64),
        ("q_lo", vp), ("k_lo", vp),
        ("gate", vp), ("gate_stride", i64 * 3),
    ]


class GridAttentionParams(ctypes.Structure):
    """Mirror of struct af3_grid_attention_params."""
    _fields_ = [
        ("pair", vp), ("pair_stride", i64 * 2),
        ("q_proj", vp), ("k_proj", vp), ("v_proj", vp), ("gating_query", vp),
        ("bias", vp), ("bias_stride", i64 * 2), ("bias_dtype", i32), ("dtype", i32),
        ("key_mask", vp), ("key_mask_stride_b", i64),
        ("out", vp), ("out_stride", i64 * 2),
        ("B", i64), ("N", i64), ("C", i64), ("head", i64),
        ("workspace", vp), ("workspace_bytes", i64),
    ]


QKV_SCRATCH_FLOATS = 768   # AF3_QKV_SCRATCH_FLOATS

# name -> (restype, argtypes); every symbol include/af3_dpa.h declares
SYMBOLS = {
    "af3_dpa_forward": (ctypes.c_int, [ctypes.POINTER(DpaParams), vp]),
    "af3_dpa_forward_static_scratch": (ctypes.c_int, [ctypes.POINTER(DpaParams), vp]),
    "af3_dpa_select_kernel": (ctypes.c_int, [ctypes.POINTER(DpaParams)]),
    "af3_dpa_workspace_bytes": (ctypes.c_int64, [ctypes.POINTER(DpaParams)]),
    "af3_grid_attention_forward": (ctypes.c_int, [ctypes.POINTER(GridAttentionParams), vp]),
    "af3_grid_attention_workspace_bytes": (ctypes.c_int64, [ctypes.POINTER(GridAttentionParams)]),
    "af3_grid_attention_supported": (ctypes.c_int, [ctypes.POINTER(GridAttentionParams)]),
    "af3_layernorm_pair_bias": (ctypes.c_int, [vp, ctypes.POINTER(i64), vp, vp, f32, vp, vp, vp, ctypes.POINTER(i64), i64, i64, i64, i64, i32, vp]),
    "af3_gated_linear_unit": (ctypes.c_int, [vp, vp, vp, i64, i64, i64, i32, vp]),
    "af3_silu_mul": (ctypes.c_int, [vp, vp, i64, i64, i32, vp]),
    "af3_linear": (ctypes.c_int, [vp, vp, vp, i64, i64, i64, i32, vp]),
    "af3_convert": (ctypes.c_int, [vp, i32, vp, i32, i64, vp]),
    "af3_amax": (ctypes.c_int, [vp, i32, i64, vp, vp]),
    "af3_quantize_fp8_e4m3": (ctypes.c_int, [vp, i32, vp, i64, i64, i64, i32, i64, i64, f32, vp, vp, vp, vp]),
    "af3_quantize_qkv_fp8_e4m3": (ctypes.c_int, [vp, vp, vp, i32, i64, i64, i64, i64, f32, vp, vp, vp, i64, vp, vp, vp, vp, vp]),
    "af3_pad_nd": (ctypes.c_int, [vp, vp, i32, ctypes.POINTER(i64), ctypes.POINTER(i64), ctypes.POINTER(i64), i32, ctypes.c_uint32, vp]),
    "af3_vnni_repack_bf16": (ctypes.c_int, [vp, vp, i64, i64, i64, vp]),
    "af3_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "af3_abi_version": (ctypes.c_int, []),
}

_lib = None


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m af3_kernels_amd.build` (hipcc, gfx950). "
                "There is no CPU or PyTorch fallback for these ops.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        if lib.af3_abi_version() != ABI_VERSION:
            raise ImportError(f"{LIB_PATH} has ABI version {lib.af3_abi_version()}, this package expects {ABI_VERSION}: rebuild it")
        _lib = lib
    return _lib


def check(status: int, what: str):
    if status != 0:
        msg = load().af3_status_string(status).decode()
        exc = ValueError if status in (-2, -3, -4, -5, -7, -9) else RuntimeError
        raise exc(f"{what}: {msg} (af3_status {status})")
