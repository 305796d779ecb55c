"""ctypes loader for the CPU oracle (oracle/af3_oracle.c).

TEST INFRASTRUCTURE ONLY: import this from tests/, from the smoke check and from the
CPU-baseline leg of the benchmark, never from the shipped package.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libaf3_oracle.so")

F32, BF16 = 0, 1


def build(force: bool = False) -> str:
    src = os.path.join(_HERE, "af3_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _SO


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        fp = ctypes.POINTER(ctypes.c_float)
        u8 = ctypes.POINTER(ctypes.c_uint8)
        u16 = ctypes.POINTER(ctypes.c_uint16)
        i64 = ctypes.c_int64
        L.af3o_dpa_reference.argtypes = [fp, fp, fp, fp, u8, fp, i64, i64, i64, i64, ctypes.c_int, ctypes.c_int, i64, i64]
        L.af3o_dpa_reference.restype = ctypes.c_int
        L.af3o_dpa_formula.argtypes = [fp, fp, fp, fp, u8, fp, i64, i64, i64, i64]
        L.af3o_dpa_formula.restype = ctypes.c_int
        L.af3o_convert_f32_to_bf16.argtypes = [fp, u16, i64]
        L.af3o_convert_bf16_to_f32.argtypes = [u16, fp, i64]
        L.af3o_quantize_e4m3.argtypes = [fp, u8, i64]
        L.af3o_quantize_e4m3.restype = ctypes.c_float
        L.af3o_quantize_e4m3_pow2.argtypes = [fp, u8, i64, ctypes.c_float]
        L.af3o_quantize_e4m3_pow2.restype = ctypes.c_float
        L.af3o_dequantize_e4m3.argtypes = [u8, fp, i64, ctypes.c_float]
        L.af3o_convert_f32_to_e5m2.argtypes = [fp, u8, i64, ctypes.c_int]
        L.af3o_convert_e5m2_to_f32.argtypes = [u8, fp, i64]
        L.af3o_f32_to_e4m3_bits.argtypes = [ctypes.c_float]
        L.af3o_f32_to_e4m3_bits.restype = ctypes.c_uint8
        L.af3o_e4m3_bits_to_f32.argtypes = [ctypes.c_uint8]
        L.af3o_e4m3_bits_to_f32.restype = ctypes.c_float
        L.af3o_vnni_repack.argtypes = [u16, u16, i64, i64, i64]
        L.af3o_vnni_repack.restype = ctypes.c_int
        L.af3o_pad_2d.argtypes = [fp, fp, i64, i64, i64, i64, ctypes.c_float]
        L.af3o_softmax_fwd.argtypes = [fp, fp, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        L.af3o_brgemm.argtypes = [fp, fp, fp] + [ctypes.c_int] * 8
        L.af3o_fused_attention_reference.argtypes = [fp, u8, fp, fp, fp, fp, fp, fp, fp, fp, i64, i64, i64, i64, ctypes.c_int, i64]
        L.af3o_fused_attention_reference.restype = ctypes.c_int
        L.af3o_fused_attention_formula.argtypes = [fp, u8, fp, fp, fp, fp, fp, fp, fp, fp, i64, i64, i64, i64]
        L.af3o_fused_attention_formula.restype = ctypes.c_int
        L.af3o_layernorm_pair_bias.argtypes = [fp, fp, fp, fp, ctypes.c_double, fp, fp, i64, i64, i64, ctypes.c_int]
        L.af3o_layernorm_pair_bias.restype = ctypes.c_int
        L.af3o_gated_linear_unit.argtypes = [fp, fp, fp, i64, i64, i64, ctypes.c_int]
        L.af3o_gated_linear_unit.restype = ctypes.c_int
        _lib = L
    return _lib


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _keep(mask, B, L):
    """Lift a user mask (1-D [L] or 2-D [B,L], truthy = attend) to contiguous [B,L] bytes,
    broadcasting a 1-D mask over the batch like examples/dot_product_attention.py:33-37."""
    m = np.asarray(mask).astype(bool)
    if m.ndim == 1:
        m = np.broadcast_to(m[None, :], (B, L))
    m = np.ascontiguousarray(m.reshape(B, L).astype(np.uint8))
    return m, m.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))


def dpa_reference(q, k, v, mask, bias, dtype=F32, use_flash=False, BLK_SZ=128, FLASH_SZ=1024):
    """Restatement of dot_product_attention_impl<T> (dot_product_attention.cpp:25-198).
    Inputs are float32 numpy arrays whose values are already representable in T."""
    B, H, L, D = q.shape
    q, qp = _f(q); k, kp = _f(k); v, vp = _f(v); bias, bp = _f(bias)
    m, mp = _keep(mask, B, L)
    out = np.empty((B, H, L, D), np.float32)
    rc = lib().af3o_dpa_reference(qp, kp, vp, bp, mp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)),
                                  B, H, L, D, dtype, int(bool(use_flash)), BLK_SZ, FLASH_SZ)
    if rc != 0:
        raise MemoryError("af3o_dpa_reference failed")
    return out


def dpa_formula(q, k, v, mask, bias):
    """examples/dot_product_attention.py:20-43 evaluated in double precision."""
    B, H, L, D = q.shape
    q, qp = _f(q); k, kp = _f(k); v, vp = _f(v); bias, bp = _f(bias)
    m, mp = _keep(mask, B, L)
    out = np.empty((B, H, L, D), np.float32)
    rc = lib().af3o_dpa_formula(qp, kp, vp, bp, mp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), B, H, L, D)
    if rc != 0:
        raise MemoryError("af3o_dpa_formula failed")
    return out


def _fused(fn, x, mask, bias, wq, wk, wv, wg, wo, qbias, head, extra):
    x = np.asarray(x, dtype=np.float32)
    squeeze = x.ndim == 2                      # the diffusion op has no batch axis: [N, C]
    if squeeze:
        x = x[None]
    B, L, C = x.shape
    x, xp = _f(x); bias, bp = _f(bias)
    ws = [_f(w) for w in (wq, wk, wv, wg)]
    null = ctypes.POINTER(ctypes.c_float)()
    wo_a, wo_p = _f(wo) if wo is not None else (None, null)
    qb_a, qb_p = _f(qbias) if qbias is not None else (None, null)
    m, mp = _keep(mask, B, L)
    out = np.empty((B, L, C), np.float32)
    rc = fn(xp, mp, bp, ws[0][1], ws[1][1], ws[2][1], ws[3][1], wo_p, qb_p, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), B, L, C, head, *extra)
    if rc != 0:
        raise MemoryError("fused attention oracle failed")
    return out[0] if squeeze else out


def fused_attention_reference(x, mask, bias, wq, wk, wv, wg, wo=None, qbias=None, head=4, dtype=BF16, BLK_SZ=128):
    """Restatement of _attention_impl<T> (wo given; dot_product_attention.cpp:200-378) and of
    self_attention_impl<T> (x [N, C], qbias; :380-543) with the reference's roundings to T.
    Weights are weight^T in natural [C_in, C_out] layout; head j uses output columns j*K .. j*K+K-1."""
    return _fused(lib().af3o_fused_attention_reference, x, mask, bias, wq, wk, wv, wg, wo, qbias, head, (dtype, BLK_SZ))


def fused_attention_formula(x, mask, bias, wq, wk, wv, wg, wo=None, qbias=None, head=4):
    """The torch modules of examples/grid_self_attention.py:46-94 (after LayerNorm and bias projection)
    and examples/self_attention.py:64-96 in double precision."""
    return _fused(lib().af3o_fused_attention_formula, x, mask, bias, wq, wk, wv, wg, wo, qbias, head, ())


def layernorm_pair_bias(pair, gamma, beta, wb, eps=1e-5, round_bf16=False):
    """LayerNorm over the last axis of pair [..., C] and the per-head bias projection with wb [H, C] (nn.Linear weight), in
    double precision (src/af3_kernels/Attention.py:51-52).  Returns (normed [..., C], bias [H, ...])."""
    pair = np.asarray(pair, dtype=np.float32)
    lead, C = pair.shape[:-1], pair.shape[-1]
    x, xp = _f(pair.reshape(-1, C))
    g, gp = _f(gamma); b, bp = _f(beta); w, wp = _f(wb)
    H, T = w.shape[0], x.shape[0]
    normed, bias = np.empty((T, C), np.float32), np.empty((H, T), np.float32)
    fpt = ctypes.POINTER(ctypes.c_float)
    lib().af3o_layernorm_pair_bias(xp, gp, bp, wp, float(eps), normed.ctypes.data_as(fpt), bias.ctypes.data_as(fpt), T, C, H, int(bool(round_bf16)))
    return normed.reshape(*lead, C), bias.reshape(H, *lead)


def gated_linear_unit(x, weight, round_bf16=False):
    """silu(x @ W[:, :N]) * (x @ W[:, N:]) for x [..., K], weight [K, 2N] (examples/gated_linear_unit.py:18-22), in double
    precision, or with the reference's bf16 roundings (src/csrc/gated_linear_unit.cpp:56-61) when round_bf16."""
    x = np.asarray(x, dtype=np.float32)
    lead, K = x.shape[:-1], x.shape[-1]
    x2, xp = _f(x.reshape(-1, K))
    w, wp = _f(weight)
    N = w.shape[1] // 2
    out = np.empty((x2.shape[0], N), np.float32)
    lib().af3o_gated_linear_unit(xp, wp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), x2.shape[0], K, N, int(bool(round_bf16)))
    return out.reshape(*lead, N)


def f32_to_bf16_bits(x):
    x, xp = _f(x)
    out = np.empty(x.shape, np.uint16)
    lib().af3o_convert_f32_to_bf16(xp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), x.size)
    return out


def bf16_bits_to_f32(h):
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().af3o_convert_bf16_to_f32(h.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), h.size)
    return out


def round_bf16(x):
    return bf16_bits_to_f32(f32_to_bf16_bits(x))


def f32_to_e5m2_bits(x, reference_rule=False):
    """fp32 -> e5m2 bits: one rounding to nearest even with overflow to infinity (the shipped converter's rule), or with
    reference_rule the two-step rule of the reference's _mm_convert_ps_bf8 (fp16 nearest-even, then the low byte dropped)."""
    x, xp = _f(x)
    out = np.empty(x.shape, np.uint8)
    lib().af3o_convert_f32_to_e5m2(xp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), x.size, int(bool(reference_rule)))
    return out


def e5m2_bits_to_f32(b):
    b = np.ascontiguousarray(b, np.uint8)
    out = np.empty(b.shape, np.float32)
    lib().af3o_convert_e5m2_to_f32(b.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), b.size)
    return out


def quantize_e4m3(x):
    """Returns (bits uint8, scale) with scale = 448/amax."""
    x, xp = _f(x)
    out = np.empty(x.shape, np.uint8)
    scale = lib().af3o_quantize_e4m3(xp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), x.size)
    return out, float(scale)


def quantize_e4m3_pow2(x, pre_scale=1.0):
    """Returns (bits uint8, scale) of the shipped quantiser's rule: scale = 2^floor(log2(448 / (amax * |pre_scale|)))
    (1 when amax is 0), bits = e4m3(x * pre_scale * scale)."""
    x, xp = _f(x)
    bits = np.empty(x.shape, np.uint8)
    scale = lib().af3o_quantize_e4m3_pow2(xp, bits.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), x.size, pre_scale)
    return bits, float(scale)


def fake_quantize_e4m3_pow2(x, pre_scale=1.0):
    """x -> e4m3 with the shipped quantiser's power-of-two per-tensor scale -> back to float32
    (including the pre_scale): what the fp8 kernels actually see."""
    bits, scale = quantize_e4m3_pow2(x, pre_scale)
    return dequantize_e4m3(bits, 1.0 / scale)


def dequantize_e4m3(bits, inv_scale=1.0):
    bits = np.ascontiguousarray(bits, dtype=np.uint8)
    out = np.empty(bits.shape, np.float32)
    lib().af3o_dequantize_e4m3(bits.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), bits.size, inv_scale)
    return out


def vnni_repack(bits, blk=0):
    bits = np.ascontiguousarray(bits, dtype=np.uint16)
    M, N = bits.shape
    out = np.empty((M, N), np.uint16)
    rc = lib().af3o_vnni_repack(bits.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint16)), M, N, blk)
    if rc != 0:
        raise ValueError("N must be divisible by BLK_SZ and M even")
    return out


def pad_2d(x, prows, pcols, init=0.0):
    x, xp = _f(x)
    out = np.empty((prows, pcols), np.float32)
    lib().af3o_pad_2d(xp, out.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), x.shape[0], x.shape[1], prows, pcols, init)
    return out
