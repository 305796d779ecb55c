"""Host side of the drop-in: argument preparation that mirrors the reference's Python wrapper,
torch custom ops, and the ctypes calls into libaf3_dpa.so.

PyTorch is used for device memory and streams only; every computation below happens in the
HIP library.  CPU tensors are rejected: there is no CPU or eager fallback.
"""
import ctypes
import threading
import math
from typing import Optional

import torch

from . import _lib
from ._lib import AF3_BF16, AF3_F32, AF3_FP8_E4M3, AF3_FP8_E5M2, DpaParams

_DTYPE_CODE = {torch.float32: AF3_F32, torch.bfloat16: AF3_BF16}
if hasattr(torch, "float8_e4m3fn"):
    _DTYPE_CODE[torch.float8_e4m3fn] = AF3_FP8_E4M3
if hasattr(torch, "float8_e5m2"):
    _DTYPE_CODE[torch.float8_e5m2] = AF3_FP8_E5M2
KERNEL_NAMES = {0: "fp32_fma", 1: "bf16_mfma", 2: "fp8_mfma", 3: "fp32_mfma"}


def _stream_ptr(device) -> int:
    """Raw handle of torch's current stream on `device` (the short route: building a torch.cuda.Stream object
    per call costs several microseconds, which a small attention call notices)."""
    return torch._C._cuda_getCurrentRawStream(device.index if device.index is not None else torch.cuda.current_device())


class _on_device:
    """`with torch.cuda.device(d)` that does nothing when d is already the current device."""
    __slots__ = ("idx", "prev")

    def __init__(self, device):
        self.idx = device.index

    def __enter__(self):
        self.prev = None
        if self.idx is not None and self.idx != torch.cuda.current_device():
            self.prev = torch.cuda.current_device()
            torch.cuda.set_device(self.idx)

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


def _require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "af3_kernels_amd ops take ROCm device tensors only (got a CPU tensor); there is no CPU fallback")


def _inner_contig(t: torch.Tensor) -> torch.Tensor:
    return t if t.stride(-1) == 1 else t.contiguous()


# ------------------------------------------------------------------------------------------
# timers: the role of reset_debug_timers / print_debug_timers (src/csrc/init.cpp:145-216) --
# per-op GPU milliseconds and TFLOP/s -- is played by HIP events recorded around each call.
# ------------------------------------------------------------------------------------------
class _Timers:
    def __init__(self):
        self.enabled = False
        self.reset()

    def reset(self):
        self.calls = 0
        self.flops = 0.0
        self.ms = 0.0
        self.pending = []

    def record(self, start, end, flops):
        self.pending.append((start, end))
        self.calls += 1
        self.flops += flops
        if len(self.pending) >= 1024:
            self.fold()

    def fold(self):
        if self.pending:
            self.pending[-1][1].synchronize()
            self.ms += sum(s.elapsed_time(e) for s, e in self.pending)
            self.pending = []


_timers = _Timers()


def reset_debug_timers():
    """Reference: src/af3_kernels/__init__.py:126-127.  Clears the accumulated GPU time and
    switches per-call event timing on."""
    _timers.reset()
    _timers.enabled = True


def print_debug_timers(tid=0, detailed=True):
    """Reference: src/af3_kernels/__init__.py:130-131.  Prints calls, GPU ms and TFLOP/s of
    dot_product_attention since the last reset (`tid` is accepted for signature parity: the
    GPU has no per-thread timers)."""
    _timers.fold()
    tf = _timers.flops / (_timers.ms * 1e-3) / 1e12 if _timers.ms > 0 else 0.0
    print(f"af3_kernels_amd timers: dot_product_attention calls={_timers.calls} gpu_ms={_timers.ms:.4f} "
          f"GF={_timers.flops / 1e9:.3f} TF/s={tf:.3f}")


def print_debug_thread_imbalance():
    """Reference: src/af3_kernels/__init__.py:134-135.  OpenMP thread imbalance has no GPU
    counterpart; prints the same totals as print_debug_timers."""
    print_debug_timers()


# ------------------------------------------------------------------------------------------
# attention
# ------------------------------------------------------------------------------------------
_PARAM_TEMPLATES = {}   # layout of a call (shapes, strides, dtypes, flags) -> bytes of an af3_dpa_params block with everything but the addresses
_PARAM_TEMPLATES_LOCK = threading.Lock()   # taken on a miss only: values are immutable bytes, a hit needs no lock


def _fill_params(q, k, v, keep, bias, out, mma_dtype, force_generic, descales=None, softmax_scale=None, v_transposed=False, gate=None) -> DpaParams:
    """The argument block of one call.  Everything that depends on the layout alone is filled once per layout and copied
    from a byte template afterwards (building the ctypes arrays anew costs more host time than a small call's kernel runs);
    only the addresses are set per call."""
    key = (q.shape, q.stride(), k.stride(), v.stride(), out.stride(), q.dtype, out.dtype, mma_dtype, bool(force_generic), _rows_kernel_hint, softmax_scale,
           None if bias is None else (bias.stride(0), bias.stride(1), bias.dtype),
           None if keep is None else (keep.shape[0], keep.stride(0)),
           None if gate is None else gate.stride())
    template = _PARAM_TEMPLATES.get(key)
    if template is None:
        B, H, L, D = q.shape
        t = DpaParams()
        t.B, t.H, t.L, t.D = B, H, L, D
        t.q_stride = (ctypes.c_int64 * 3)(*q.stride()[:3])
        t.k_stride = (ctypes.c_int64 * 3)(*k.stride()[:3])
        t.v_stride = (ctypes.c_int64 * 3)(*v.stride()[:3])
        t.out_stride = (ctypes.c_int64 * 3)(*out.stride()[:3])
        if bias is not None:
            t.bias_stride = (ctypes.c_int64 * 2)(bias.stride(0), bias.stride(1))
            t.bias_dtype = _DTYPE_CODE[bias.dtype]
        if keep is not None:
            t.key_mask_stride_b = 0 if keep.shape[0] == 1 else keep.stride(0)
        t.io_dtype = _DTYPE_CODE[q.dtype]
        t.out_dtype = _DTYPE_CODE[out.dtype]
        t.mma_dtype = mma_dtype
        t.softmax_scale = float(D) ** -0.5 if softmax_scale is None else softmax_scale
        t.q_descale = t.k_descale = t.v_descale = 1.0
        t.force_generic = int(bool(force_generic))
        t.reserved = _rows_kernel_hint
        if gate is not None:
            t.gate_stride = (ctypes.c_int64 * 3)(*gate.stride()[:3])
        template = bytes(t)
        with _PARAM_TEMPLATES_LOCK:
            if len(_PARAM_TEMPLATES) >= 256:
                _PARAM_TEMPLATES.clear()
            _PARAM_TEMPLATES[key] = template
    p = DpaParams.from_buffer_copy(template)
    p.q, p.k, p.v, p.out = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    if bias is not None:
        p.bias = bias.data_ptr()
    if keep is not None:
        p.key_mask = keep.data_ptr()
    if descales is not None:
        p.device_descales = descales.data_ptr()
    if gate is not None:
        p.gate = gate.data_ptr()
    return p


def _check_shapes(q, k, v, keep, bias, v_transposed=False):
    if q.dim() != 4:
        raise ValueError(f"q must be [B, H, L, D], got {tuple(q.shape)}")
    B, H, L, D = q.shape
    vshape = (B, H, D, L) if v_transposed else (B, H, L, D)
    if tuple(k.shape) != (B, H, L, D) or tuple(v.shape[:2]) != (B, H) or (not v_transposed and tuple(v.shape) != vshape):
        raise ValueError(f"k and v must have q's shape {tuple(q.shape)} (q_len == k_len), got {tuple(k.shape)} and {tuple(v.shape)}")
    if bias is not None:
        if bias.dim() != 3 or bias.shape[0] != H or bias.shape[1] < L or bias.shape[2] < L:
            raise ValueError(f"bias must be [H, L, L] (or padded [H, M, M]) with H={H}, L={L}, got {tuple(bias.shape)}")
    if keep is not None:
        if keep.dim() != 2 or keep.shape[1] != L or keep.shape[0] not in (1, B):
            raise ValueError(f"mask must be [L] or [B, L] with B={B}, L={L}, got {tuple(keep.shape)}")


_exact_bias = False
_rows_kernel_hint = 0


def set_rows_kernel(mode: str) -> str:
    """Kernel choice for batched bf16 calls that the shared-bias kernel (two to four batch rows per wavefront) can take
    (head_dim <= 32, at least two batch rows, L <= 4096): "auto" (default: taken when the launch suits it), "always" or
    "never" (testing aids).  Process-wide, like the reference's module-level switches.  Returns the previous mode."""
    global _rows_kernel_hint
    names = ("auto", "always", "never")
    prev, _rows_kernel_hint = names[_rows_kernel_hint], names.index(mode)
    return prev


def set_exact_bias(flag: bool) -> bool:
    """With True, batched bf16 calls pass no bias workspace: the bias is read in place and added exactly.  That only
    matters for calls the one-row kernel serves (head_dim 48/64, small launches), whose workspace holds
    fp16(bias * log2 e) -- a rounding error of at most 2^-11 * |bias| * log2 e per logit: irrelevant for pair biases of
    ordinary size, 2 % of a softmax weight at |bias| = 40; the shared-bias kernel's workspace is fp32 and exact.
    Slower for B >= 2.  Returns the previous setting."""
    global _exact_bias
    prev, _exact_bias = _exact_bias, bool(flag)
    return prev


def _dpa_forward_impl(q, k, v, keep, bias, mma_dtype: int, force_generic: bool, gate=None, out=None) -> torch.Tensor:
    """gate: optional [B,H,L,D] pre-activation values, the result is multiplied by sigmoid(gate) in the
    kernel's epilogue; out: optional preallocated (possibly strided, innermost stride 1) result view."""
    _require_device(q, k, v, keep, bias, gate, out)
    q, k, v = _inner_contig(q), _inner_contig(k), _inner_contig(v)
    if gate is not None and (gate.stride(-1) != 1 or tuple(gate.shape) != tuple(q.shape) or gate.dtype != q.dtype):
        raise ValueError("gate must have q's shape and dtype with a unit innermost stride")
    if out is not None and (out.stride(-1) != 1 or tuple(out.shape) != tuple(q.shape)):
        raise ValueError("out must have q's shape with a unit innermost stride")
    if bias is not None:
        bias = _inner_contig(bias)
    if keep is not None:
        keep = _inner_contig(keep)
    _check_shapes(q, k, v, keep, bias)
    if out is None:
        out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    if q.numel() == 0:
        return out
    p = _fill_params(q, k, v, keep, bias, out, mma_dtype, force_generic, gate=gate)
    lib = _lib.load()
    ws_bytes = lib.af3_dpa_workspace_bytes(ctypes.byref(p))
    if ws_bytes > 0 and not _exact_bias:
        # scratch for the kernel's bias rewrite; torch's caching allocator makes this a pointer bump
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device)
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws_bytes
    with _on_device(q.device):
        if _timers.enabled:
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
        _lib.check(lib.af3_dpa_forward(ctypes.byref(p), _stream_ptr(q.device)), "af3_dpa_forward")
        if _timers.enabled:
            e.record()
            B, H, L, D = q.shape
            _timers.record(s, e, 4.0 * B * H * L * L * D)
    return out


@torch.library.custom_op("af3_kernels::dpa_forward", mutates_args=())
def _dpa_forward_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, key_mask: Optional[torch.Tensor], bias: Optional[torch.Tensor],
                    mma_dtype: int, force_generic: bool) -> torch.Tensor:
    """Lean op: key_mask is uint8 [1|B, L], non-zero = attend."""
    return _dpa_forward_impl(q, k, v, key_mask, bias, mma_dtype, force_generic)


@_dpa_forward_op.register_fake
def _(q, k, v, key_mask, bias, mma_dtype, force_generic):
    return torch.empty_like(q)


@torch.library.custom_op("af3_kernels::dot_product_attention", mutates_args=())
def _dot_product_attention_op(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor, bias: torch.Tensor,
                              use_flash_attention: bool, BLK_SZ: int, FLASH_SZ: int) -> torch.Tensor:
    """Same argument list as the reference's native entry point (src/csrc/init.cpp:349-351,
    src/csrc/dot_product_attention.h:25-32): `mask` arrives already inverted and cast to q's
    dtype, shape [B|1, 1, 1, L], 1.0 = dropped key.  use_flash_attention, BLK_SZ and FLASH_SZ are
    CPU cache-blocking hints and change nothing here."""
    L = q.shape[2]
    keep = (mask.reshape(-1, L) == 0).to(torch.uint8)
    code = _DTYPE_CODE.get(q.dtype)
    if code is None:
        raise ValueError(f"unsupported dtype {q.dtype}: float32 or bfloat16")
    return _dpa_forward_impl(q, k.to(q.dtype), v.to(q.dtype), keep, bias.to(q.dtype), code, False)


@_dot_product_attention_op.register_fake
def _(q, k, v, mask, bias, use_flash_attention, BLK_SZ, FLASH_SZ):
    return torch.empty_like(q)


def _lift_mask(mask: Optional[torch.Tensor], L: int) -> Optional[torch.Tensor]:
    """Rank-lifting of src/af3_kernels/__init__.py:41-44 without the inversion: returns uint8
    [1|B, L], non-zero = attend.  A bool mask is reinterpreted, not copied."""
    if mask is None:
        return None
    if mask.dim() == 1:
        mask = mask[None, :]
    elif mask.dim() == 4:
        mask = mask.reshape(mask.shape[0], mask.shape[-1])
    elif mask.dim() != 2:
        raise ValueError(f"mask must have 1, 2 or 4 dimensions, got {mask.dim()}")
    if mask.dtype != torch.bool:
        mask = mask.to(dtype=torch.bool)
    return _inner_contig(mask).view(torch.uint8)


def dot_product_attention_cpp(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    mask: torch.Tensor,
    bias: torch.Tensor,
    use_flash_attention: bool = False,
    BLK_SZ: int = 128,
    FLASH_SZ: int = 1024,
) -> torch.Tensor:
    """softmax(q.k^T * D^-1/2 + bias, mask) . v  -- drop-in for the reference's
    af3_kernels.dot_product_attention_cpp (src/af3_kernels/__init__.py:31-52).

    q, k, v [B,H,L,D]; bias [H,L,L] (or pre-padded [H,M,M]); mask [L], [B,L] or [B,1,1,L],
    truthy = attend.  float32 inputs run in fp32 FMA arithmetic, bfloat16 inputs on the bf16
    matrix cores with fp32 accumulation.  As in the reference, k, v and bias are cast to q's
    dtype.  Unlike the reference, q is left untouched and a fresh tensor is returned; a 1-D
    mask is broadcast over the batch (the harness semantics, examples/dot_product_attention.py:
    34-37).  use_flash_attention / BLK_SZ / FLASH_SZ are accepted and ignored: they tune CPU
    cache blocking and never change results (the kernel is always an online-softmax kernel)."""
    code = _DTYPE_CODE.get(q.dtype)
    if code not in (AF3_F32, AF3_BF16):
        raise ValueError(f"unsupported dtype {q.dtype}: float32 or bfloat16 (use dot_product_attention_fp8 for the fp8 path)")
    dtype = q.dtype
    keep = _lift_mask(mask, q.shape[2]) if mask is not None else None
    # (a cast to the dtype a tensor already has returns the tensor, but the call alone costs a microsecond of a 20-us call)
    if bias is not None and bias.dtype != dtype:
        bias = bias.to(dtype)
    if k.dtype != dtype:
        k = k.to(dtype)
    if v.dtype != dtype:
        v = v.to(dtype)
    # (straight into the implementation: the registered op torch.ops.af3_kernels.dpa_forward is the same function
    # behind torch's dispatcher, whose per-call cost is comparable to a small attention kernel)
    return _dpa_forward_impl(q, k, v, keep, bias, code, False)


def selected_kernel(q, k, v, mask, bias, force_generic=False) -> str:
    """Name of the kernel dot_product_attention_cpp would run for these tensors."""
    keep = _lift_mask(mask, q.shape[2]) if mask is not None else None
    out = torch.empty_like(q)
    p = _fill_params(_inner_contig(q), _inner_contig(k), _inner_contig(v), keep, bias, out, _DTYPE_CODE[q.dtype], force_generic)
    rc = _lib.load().af3_dpa_select_kernel(ctypes.byref(p))
    _lib.check(min(rc, 0), "af3_dpa_select_kernel")
    return KERNEL_NAMES[rc]


# ------------------------------------------------------------------------------------------
# casts and per-tensor fp8 scaling
# ------------------------------------------------------------------------------------------
def convert(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Element-wise cast on the device (tpp::ConvertTPP, src/csrc/xsmm_functors.h:838-885):
    f32<->bf16 (round to nearest even), e4m3 -> f32 / bf16, and e5m2 <-> f32 / bf16 (the reference's bf8 helpers,
    src/csrc/xsmm_functors.h:211-217; to e5m2: round to nearest even, overflow to infinity, like torch.float8_e5m2)."""
    _require_device(x)
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    with _on_device(x.device):
        _lib.check(_lib.load().af3_convert(x.data_ptr(), _DTYPE_CODE[x.dtype], out.data_ptr(), _DTYPE_CODE[dtype], x.numel(),
                                           _stream_ptr(x.device)), "af3_convert")
    return out


def quantize_fp8_e4m3(x: torch.Tensor, pre_scale: float = 1.0, transpose_last2: bool = False, descale_out: Optional[torch.Tensor] = None,
                      with_residual: bool = False, amax_buf: Optional[torch.Tensor] = None):
    """Per-tensor scaled quantisation to OCP e4m3: returns (fp8 tensor, descale) where descale is
    a 1-element device float and real ~= fp8 * descale.  The scale is the largest power of two
    that keeps amax * pre_scale <= 448.  With transpose_last2 the last two axes are swapped in
    the output and the new innermost axis is padded (with zeros) to a multiple of 16 bytes.  With
    with_residual a third value is returned: e4m3(x * pre_scale * scale - fp8), the rounding error
    at the same scale.  amax_buf: optional 1-element device float that already holds 0 (saves the
    fill a fresh one needs)."""
    _require_device(x)
    if x.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("quantize_fp8_e4m3 takes float32 or bfloat16")
    x = x.contiguous()
    rows_per_matrix, cols = x.shape[-2], x.shape[-1]
    rows = x.numel() // cols
    lib = _lib.load()
    amax = amax_buf if amax_buf is not None else torch.zeros(1, dtype=torch.float32, device=x.device)
    if descale_out is None:
        descale_out = torch.empty(1, dtype=torch.float32, device=x.device)
    with _on_device(x.device):
        st = _stream_ptr(x.device)
        _lib.check(lib.af3_amax(x.data_ptr(), _DTYPE_CODE[x.dtype], x.numel(), amax.data_ptr(), st), "af3_amax")
        if transpose_last2:
            lpad = (rows_per_matrix + 15) // 16 * 16
            # (the quantiser writes the padding itself: nothing to clear)
            full = torch.empty(x.shape[:-2] + (cols, lpad), dtype=torch.float8_e4m3fn, device=x.device)
            out = full[..., :rows_per_matrix]
            full_lo = torch.empty_like(full) if with_residual else None
            lo = full_lo[..., :rows_per_matrix] if with_residual else None
            _lib.check(lib.af3_quantize_fp8_e4m3(x.data_ptr(), _DTYPE_CODE[x.dtype], full.data_ptr(), rows, cols, cols, 1, rows_per_matrix, lpad,
                                                 pre_scale, amax.data_ptr(), descale_out.data_ptr(), full_lo.data_ptr() if with_residual else None, st),
                       "af3_quantize_fp8_e4m3")
        else:
            out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
            lo = torch.empty_like(out) if with_residual else None
            _lib.check(lib.af3_quantize_fp8_e4m3(x.data_ptr(), _DTYPE_CODE[x.dtype], out.data_ptr(), rows, cols, cols, 0, 0, cols,
                                                 pre_scale, amax.data_ptr(), descale_out.data_ptr(), lo.data_ptr() if with_residual else None, st),
                       "af3_quantize_fp8_e4m3")
    return (out, descale_out, lo) if with_residual else (out, descale_out)


def dot_product_attention_fp8(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, mask: torch.Tensor, bias: torch.Tensor,
                              compensated: bool = True) -> torch.Tensor:
    """Attention with both products on the e4m3 matrix cores (fp32 accumulation): q, k, v are
    quantised per tensor (q with D^-1/2 folded in, v written transposed), the bias stays bf16,
    the output has q's dtype.  With `compensated` (default) q and k also carry their e4m3 rounding
    residuals and the logits are q8.k8 + q8.k_lo + q_lo.k8 (three e4m3 MFMAs per chunk), which is
    what keeps the result within 6e-2 of the fp32 formula; without it only q8.k8 is computed.
    No reference counterpart (the reference has no fp8 path)."""
    _require_device(q, k, v, mask, bias)
    B, H, L, D = q.shape
    if q.dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("dot_product_attention_fp8 takes float32 or bfloat16 inputs")
    if tuple(k.shape) != (B, H, L, D) or tuple(v.shape) != (B, H, L, D):
        raise ValueError(f"k and v must have q's shape {tuple(q.shape)}, got {tuple(k.shape)} and {tuple(v.shape)}")
    if D % 4 != 0:
        raise ValueError("the fp8 path needs head_dim % 4 == 0")
    q, k, v = q.contiguous(), k.to(q.dtype).contiguous(), v.to(q.dtype).contiguous()
    # one launch for the three amax reductions, one for the three quantisations (q with D^-1/2 folded in and
    # k with residuals, v transposed and padded to 16 keys)
    lpad = (L + 15) // 16 * 16
    f8 = torch.float8_e4m3fn
    q8, k8 = torch.empty(q.shape, dtype=f8, device=q.device), torch.empty(q.shape, dtype=f8, device=q.device)
    q_lo, k_lo = (torch.empty_like(q8), torch.empty_like(k8)) if compensated else (None, None)
    v8t_full = torch.empty((B, H, D, lpad), dtype=f8, device=q.device)
    v8t = v8t_full[..., :L]
    scratch = torch.empty(3 + _lib.QKV_SCRATCH_FLOATS, dtype=torch.float32, device=q.device)
    descales = scratch[0:3]
    with _on_device(q.device):
        _lib.check(_lib.load().af3_quantize_qkv_fp8_e4m3(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), _DTYPE_CODE[q.dtype], B, H, L, D, float(D) ** -0.5, q8.data_ptr(), k8.data_ptr(), v8t_full.data_ptr(), lpad,
            q_lo.data_ptr() if compensated else None, k_lo.data_ptr() if compensated else None, descales.data_ptr(), scratch[3:].data_ptr(),
            _stream_ptr(q.device)), "af3_quantize_qkv_fp8_e4m3")
    keep = _lift_mask(mask, L) if mask is not None else None
    bias = _inner_contig(bias.to(torch.bfloat16)) if bias is not None else None
    _check_shapes(q8, k8, v8t, keep, bias, v_transposed=True)
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    p = _fill_params(q8, k8, v8t, keep, bias, out, AF3_FP8_E4M3, False, descales=descales, softmax_scale=1.0)
    if compensated:
        p.q_lo, p.k_lo = q_lo.data_ptr(), k_lo.data_ptr()
    with _on_device(q.device):
        _lib.check(_lib.load().af3_dpa_forward(ctypes.byref(p), _stream_ptr(q.device)), "af3_dpa_forward(fp8)")
    return out


# ------------------------------------------------------------------------------------------
# layout helpers kept for callers of the reference's helpers
# ------------------------------------------------------------------------------------------
def pad_and_align_tensor(x: torch.Tensor, shape, need_init: bool = True, init: float = 0.0, alignment: int = 64) -> torch.Tensor:
    """Reference: src/af3_kernels/__init__.py:108-115, src/csrc/tools.cpp:42-124.  Pads x up to
    `shape` (filling with `init` when need_init) in a fresh device tensor; returns x itself when it
    already has that many elements, is contiguous and aligned (tools.cpp:78-82)."""
    _require_device(x)
    shape = tuple(int(s) for s in shape)
    if len(shape) != x.dim():
        raise ValueError("padded shape must have the tensor's rank")
    if math.prod(shape) == x.numel() and x.is_contiguous() and x.data_ptr() % alignment == 0:
        return x
    if x.dim() > 6 or x.element_size() not in (1, 2, 4):
        raise ValueError("pad_and_align_tensor supports up to 6 dimensions and 1-, 2- or 4-byte elements")
    out = torch.empty(shape, dtype=x.dtype, device=x.device)  # torch's allocator aligns to >= 256 bytes
    fill = torch.tensor([init if need_init else 0.0], dtype=x.dtype).view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[x.element_size()])
    fill_bits = int(fill.item()) & 0xFFFFFFFF
    n = x.dim()
    arr = ctypes.c_int64 * n
    with _on_device(x.device):
        _lib.check(_lib.load().af3_pad_nd(x.data_ptr(), out.data_ptr(), n, arr(*x.shape), arr(*x.stride()), arr(*shape), x.element_size(),
                                          fill_bits, _stream_ptr(x.device)), "af3_pad_nd")
    return out


def vnni_repack_tensor(x: torch.Tensor, type: int = 2, BLK_SZ: int = 0) -> torch.Tensor:
    """Reference: src/af3_kernels/__init__.py:118-123, src/csrc/tools.cpp:151-176.  bf16 [M, N] ->
    per BLK_SZ-wide column panel [N/BLK][M/2][BLK][2].  Only type 2 (XFORM_N2V) is used by the
    reference's callers and implemented here."""
    _require_device(x)
    if x.dim() != 2:
        raise ValueError("VNNI Repack only support 2D tensor")
    if x.dtype != torch.bfloat16:
        raise ValueError("VNNI Repack only support bf16 tensor")
    if not x.is_contiguous():
        raise ValueError("VNNI Repack only support contiguous tensor")
    if type != 2:
        raise ValueError("only XFORM_N2V (type=2) is implemented")
    M, N = x.shape
    out = torch.empty_like(x)
    with _on_device(x.device):
        _lib.check(_lib.load().af3_vnni_repack_bf16(x.data_ptr(), out.data_ptr(), M, N, BLK_SZ, _stream_ptr(x.device)), "af3_vnni_repack_bf16")
    return out
