"""The callers around the attention core, with the reference's names and argument lists:

    _attention_cpp         src/af3_kernels/__init__.py:55-80    -> _attention_impl      (dot_product_attention.cpp:200-378)
    self_attention_cpp     src/af3_kernels/__init__.py:83-105   -> self_attention_impl  (dot_product_attention.cpp:380-543)
    GridSelfAttentionCpp   src/af3_kernels/Attention.py:23-82   (the module around _attention_cpp)
    layernorm_pair_bias    src/af3_kernels/Attention.py:51-52   (torch ops in the reference: LayerNorm, bias projection, permute)
    gated_linear_unit_cpp  src/af3_kernels/__init__.py:21-28    -> gated_linear_unit_impl (gated_linear_unit.cpp:20-80)
    Linear                 src/af3_kernels/__init__.py:138-163  -> linear_impl            (gated_linear_unit.cpp:82-129)

On the GPU the grid op in AlphaFold 3's shape (bfloat16, 128 channels, 4 heads) is ONE kernel for the projections,
the attention and the gate (af3_grid_attention_forward: q, k, v and the gate never touch device memory) followed by
the output projection (af3_linear).  Every other shape, and the diffusion op, is three launches:
  1. ONE library GEMM for the four projections: x [rows, C] . W [C, 4C], output columns ordered
     (head, [k, v, q, gate], channel)  (hipBLASLt through torch: a plain GEMM is library territory);
  2. the attention kernel, reading q, k, v and the gate where that GEMM left them (no
     "b n (h d) -> b h n d" copies), adding bias and mask, and applying sigmoid(gate) in its
     epilogue while writing straight into the "b n (h d)" layout;
  3. the output projection (grid attention only).
Weights arrive in the layout the reference's callers produce with vnni_repack_tensor(W.T, 2, C/head)
and are unpacked once per weight set into the fused matrix (cached per live weight tensor and version).
"""
import ctypes
import threading
import weakref
from typing import Optional

import torch

from . import _lib, ops

# One workgroup of the fused kernel serves one (batch row, head) and holds a compute unit's LDS: launches with
# fewer workgroups than this leave most of the 256 compute units idle and take the three-launch path instead.
_FUSED_MIN_GROUPS = 128

_W_CACHE = {}
_W_CACHE_MAX = 64
_ATTEND_TEMPLATES = {}   # (B, N, head, K, dtype code) -> bytes of an af3_dpa_params block with the shape-dependent fields set
_CACHE_LOCK = threading.RLock()   # guards the two caches' updates (lookups of immutable values need none)


def _unpack_panels(w: torch.Tensor, head: int) -> torch.Tensor:
    """Inverse of vnni_repack_tensor(W_t, 2, K) (src/csrc/tools.cpp:151-176) for W_t = weight^T [C, C]:
    the packed tensor holds, per head j, the [C, K] column panel of W_t as [C/2][K][2] (bf16 pairs of
    consecutive input rows).  float32 weights have a pair size of 1, i.e. panels stored as [C][K]."""
    C = w.shape[0]
    K = C // head
    if w.dtype == torch.bfloat16:
        return w.reshape(head, C // 2, K, 2).permute(1, 3, 0, 2).reshape(C, C)
    return w.reshape(head, C, K).permute(1, 0, 2).reshape(C, C)


def _layout(t: torch.Tensor):
    return (t.data_ptr(), t.storage_offset(), tuple(t.shape), tuple(t.stride()), t.dtype)


def _cached(sources, extra, make):
    """make()'s result, remembered for as long as the source tensors are the same live objects at the same
    version, address and layout (an in-place update bumps the version; set_() or a resize moves the address or
    layout; a freed tensor's id may be reused by another tensor, which the weak references tell apart).
    Writes that bypass the version counter -- `weight.data.copy_(...)`, a foreign kernel writing the storage --
    cannot be seen from here: call clear_weight_cache() after them."""
    key = tuple(id(t) for t in sources) + extra
    hit = _W_CACHE.get(key)
    state = tuple((t._version,) + _layout(t) for t in sources)
    if hit is not None:
        refs, seen, value = hit
        if all(r() is t for r, t in zip(refs, sources)) and seen == state:
            return value
    value = make()                               # (outside the lock: it may launch kernels; two threads that miss together both build it)
    with _CACHE_LOCK:
        for k in [k for k, (refs, _, _) in list(_W_CACHE.items()) if any(r() is None for r in refs)]:
            _W_CACHE.pop(k, None)                # derived matrices of weights that no longer exist
        if len(_W_CACHE) >= _W_CACHE_MAX:
            _W_CACHE.clear()
        _W_CACHE[key] = (tuple(weakref.ref(t) for t in sources), state, value)
    return value


def clear_weight_cache() -> None:
    """Forgets every matrix derived from a weight tensor (the fused [4C, C] projection, the transposed output
    projection, the gated linear unit's weight^T).  Needed only after weights were overwritten in a way that
    does not bump the tensor's version counter, e.g. `module.weight.data.copy_(new)`; ordinary in-place
    updates (`copy_`, `load_state_dict`, optimiser steps) are noticed without it."""
    with _CACHE_LOCK:
        _W_CACHE.clear()


def _fused_weight(ws, head: int, dtype: torch.dtype) -> torch.Tensor:
    """The four projection matrices (q, k, v, gate: weight^T in panel layout) as ONE [4C, C] matrix for a single
    GEMM, rows (= output columns) ordered (head, [k, v, q, gate], channel): the 4K values of one token and
    head are contiguous, K and V side by side, so that every 128-byte line the attention kernel fetches
    for a key is used whole by the workgroups of that head."""
    def make():
        C = ws[0].shape[0]
        K = C // head
        q, k, v, g = (_unpack_panels(w, head).to(dtype).view(C, head, K) for w in ws)
        return torch.stack((k, v, q, g), dim=2).reshape(C, 4 * C).t().contiguous()
    return _cached(tuple(ws), (head, dtype), make)


def _q_bias_row(q_bias: torch.Tensor, head: int, dtype: torch.dtype) -> torch.Tensor:
    """[4C] row added by the projection GEMM's epilogue: q_bias in the q columns, zero elsewhere."""
    def make():
        C = q_bias.numel()
        K = C // head
        row = torch.zeros(head, 4, K, dtype=dtype, device=q_bias.device)
        row[:, 2] = q_bias.reshape(head, K).to(dtype)
        return row.view(4 * C)
    return _cached((q_bias,), (head, dtype, "q_bias"), make)


def _check_weights(C: int, head: int, ws):
    if C % head != 0:
        raise ValueError(f"channel count {C} is not divisible by head={head}")
    for w in ws:
        if w.dim() != 2 or w.shape[0] != C or w.shape[1] != C:
            raise ValueError(f"projection weights must be [{C}, {C}], got {tuple(w.shape)}")
        if not w.is_contiguous():
            raise ValueError("projection weights must be contiguous (they carry a packed layout)")


def _project(rows: torch.Tensor, ws, q_bias: Optional[torch.Tensor], head: int) -> torch.Tensor:
    """Stage 1: [rows, C] . [C, 4C] -> per token and head (k | v | q | gate).  The q bias of the diffusion op
    rides the GEMM's epilogue."""
    W = _fused_weight(ws, head, rows.dtype)
    return torch.nn.functional.linear(rows, W, None if q_bias is None else _q_bias_row(q_bias, head, rows.dtype))


def _attend(y: torch.Tensor, B: int, N: int, head: int, mask, bias) -> torch.Tensor:
    """Stage 2: the attention kernel on q, k, v and the gate where stage 1 left them -- [B, head, N, K] views of y with
    strides (N*4C, 4K, 4C, 1), no "b n (h d) -> b h n d" copies; sigmoid(gate) is applied in the kernel's epilogue and the
    result lands in "b n (h d)" order.  The argument block is filled from y's address directly: building the four views
    with tensor ops costs more host time than the kernel of a short sequence runs.  Returns [B, N, C]."""
    C = y.shape[1] // 4
    K = C // head
    if not y.is_contiguous():
        y = y.contiguous()
    out = torch.empty(B, N, C, dtype=y.dtype, device=y.device)
    if out.numel() == 0:
        return out
    keep = ops._lift_mask(mask, N) if mask is not None else None
    if keep is not None and keep.shape[0] not in (1, B):
        raise ValueError(f"mask must be [N] or [B, N] with B={B}, N={N}, got {tuple(mask.shape)}")
    if bias is not None:
        bias = ops._inner_contig(bias if bias.dtype == y.dtype else bias.to(y.dtype))
        if bias.dim() != 3 or bias.shape[0] != head or bias.shape[1] < N or bias.shape[2] < N:
            raise ValueError(f"bias must be [head, N, N] with head={head}, N={N}, got {tuple(bias.shape)}")
    code, esz, base = ops._DTYPE_CODE[y.dtype], y.element_size(), y.data_ptr()
    # everything that depends on the shape alone is filled once per shape: this runs per layer of a model, and for short
    # sequences the host side of a call costs as much as its kernels
    shape_key = (B, N, head, K, code)
    template = _ATTEND_TEMPLATES.get(shape_key)
    if template is None:
        t = _lib.DpaParams()
        strides = (ctypes.c_int64 * 3)(N * 4 * C, 4 * K, 4 * C)
        t.q_stride = t.k_stride = t.v_stride = t.gate_stride = strides
        t.out_stride = (ctypes.c_int64 * 3)(N * C, K, C)
        t.B, t.H, t.L, t.D = B, head, N, K
        t.io_dtype = t.out_dtype = t.mma_dtype = t.bias_dtype = code
        t.softmax_scale = float(K) ** -0.5
        t.q_descale = t.k_descale = t.v_descale = 1.0
        template = bytes(t)
        with _CACHE_LOCK:
            if len(_ATTEND_TEMPLATES) >= 256:
                _ATTEND_TEMPLATES.clear()
            _ATTEND_TEMPLATES[shape_key] = template
    p = _lib.DpaParams.from_buffer_copy(template)
    p.k, p.v, p.q, p.gate = base, base + K * esz, base + 2 * K * esz, base + 3 * K * esz   # per token and head: (k | v | q | gate)
    p.out = out.data_ptr()
    p.reserved = ops._rows_kernel_hint
    if bias is not None:
        p.bias = bias.data_ptr()
        p.bias_stride[0], p.bias_stride[1] = bias.stride(0), bias.stride(1)
    if keep is not None:
        p.key_mask, p.key_mask_stride_b = keep.data_ptr(), (0 if keep.shape[0] == 1 else keep.stride(0))
    lib = _lib.load()
    ws_bytes = lib.af3_dpa_workspace_bytes(ctypes.byref(p))
    if ws_bytes > 0 and not ops._exact_bias:
        scratch = torch.empty(ws_bytes, dtype=torch.uint8, device=y.device)
        p.workspace, p.workspace_bytes = scratch.data_ptr(), ws_bytes
    with ops._on_device(y.device):
        _lib.check(lib.af3_dpa_forward(ctypes.byref(p), ops._stream_ptr(y.device)), "af3_dpa_forward")
    return out


def _fused_grid_kernel(pair: torch.Tensor, mask, bias, ws, head: int) -> Optional[torch.Tensor]:
    """Projections, attention and gate in ONE kernel (af3_grid_attention_forward) when the library supports the
    shape (bfloat16, 128 channels, 4 heads, K and V of a head fit in LDS); None otherwise.  Returns [B, N, C]."""
    if ops._exact_bias or any(w.dtype != pair.dtype for w in ws):
        return None
    B, N, C = pair.shape
    if pair.stride(-1) != 1:
        pair = pair.contiguous()
    g = _lib.GridAttentionParams()
    g.pair, g.pair_stride = pair.data_ptr(), (ctypes.c_int64 * 2)(pair.stride(0), pair.stride(1))
    g.q_proj, g.k_proj, g.v_proj, g.gating_query = (w.data_ptr() for w in ws)
    g.B, g.N, g.C, g.head = B, N, C, head
    g.dtype = ops._DTYPE_CODE[pair.dtype]
    out = torch.empty(B, N, C, dtype=pair.dtype, device=pair.device)
    g.out, g.out_stride = out.data_ptr(), (ctypes.c_int64 * 2)(N * C, C)
    if bias is not None:
        bias = ops._inner_contig(bias)
        if bias.dtype not in ops._DTYPE_CODE or bias.dim() != 3 or bias.shape[0] != head or bias.shape[1] < N or bias.shape[2] < N:
            return None
        g.bias, g.bias_stride, g.bias_dtype = bias.data_ptr(), (ctypes.c_int64 * 2)(bias.stride(0), bias.stride(1)), ops._DTYPE_CODE[bias.dtype]
    keep = ops._lift_mask(mask, N) if mask is not None else None
    if keep is not None:
        if keep.shape[0] not in (1, B):
            raise ValueError(f"mask must be [N] or [B, N] with B={B}, N={N}, got {tuple(mask.shape)}")
        g.key_mask, g.key_mask_stride_b = keep.data_ptr(), (0 if keep.shape[0] == 1 else keep.stride(0))
    lib = _lib.load()
    if not lib.af3_grid_attention_supported(ctypes.byref(g)):
        return None
    ws_bytes = lib.af3_grid_attention_workspace_bytes(ctypes.byref(g))
    if ws_bytes > 0:
        scratch = torch.empty(ws_bytes, dtype=torch.uint8, device=pair.device)
        g.workspace, g.workspace_bytes = scratch.data_ptr(), ws_bytes
    with ops._on_device(pair.device):
        _lib.check(lib.af3_grid_attention_forward(ctypes.byref(g), ops._stream_ptr(pair.device)), "af3_grid_attention_forward")
    return out


def _attention_cpp(
    pair: torch.Tensor,
    mask: torch.Tensor,
    bias: torch.Tensor,
    q_proj: torch.Tensor,
    k_proj: torch.Tensor,
    v_proj: torch.Tensor,
    gating_query: torch.Tensor,
    out_proj: torch.Tensor,
    head: int,
    use_flash_attention: bool = False,  # unused, as in the reference
    BLK_SZ: int = 128,                   # CPU tile size in the reference; no meaning here
    FLASH_SZ: int = 1024,                # unused, as in the reference
) -> torch.Tensor:
    """Grid / triangle self-attention on already normalised pair rows:
        q, k, v, g = pair . Wq, Wk, Wv, Wg  (per head);  out = (softmax(q k^T K^-1/2 + bias, mask) v * sigmoid(g)) . Wout
    pair [B, N, C]; mask [B, N] or [N] (truthy = attend); bias [head, N, N]; q_proj, k_proj, v_proj,
    gating_query: weight^T packed with vnni_repack_tensor(., 2, C/head); out_proj: weight^T [C, C].
    Returns [B, N, C] in pair's dtype (bfloat16 or float32)."""
    ops._require_device(pair, mask, bias, q_proj, k_proj, v_proj, gating_query, out_proj)
    if pair.dim() != 3:
        raise ValueError(f"pair must be [B, N, C], got {tuple(pair.shape)}")
    B, N, C = pair.shape
    _check_weights(C, head, (q_proj, k_proj, v_proj, gating_query, out_proj))
    dtype = pair.dtype
    code = ops._DTYPE_CODE.get(dtype)
    if code not in (ops.AF3_F32, ops.AF3_BF16):
        raise ValueError(f"unsupported dtype {dtype}: float32 or bfloat16")
    ws = (q_proj, k_proj, v_proj, gating_query)
    gated = _fused_grid_kernel(pair, mask, bias, ws, head) if B * head >= _FUSED_MIN_GROUPS else None
    if gated is None:
        gated = _attend(_project(pair.reshape(B * N, C), ws, None, head), B, N, head, mask, bias)
    rows = gated.view(B * N, C)
    if out_proj.dtype == dtype and _narrow_linear_ok(rows, C):
        w = _cached((out_proj,), ("out_proj",), lambda: out_proj.t().contiguous())      # nn.Linear layout [out, in]
        return _linear_rows(rows, w).view(B, N, C)
    return torch.matmul(rows, out_proj.to(dtype)).view(B, N, C)


def self_attention_cpp(
    pair: torch.Tensor,
    mask: torch.Tensor,
    bias: torch.Tensor,
    q_proj: torch.Tensor,
    q_bias: torch.Tensor,
    k_proj: torch.Tensor,
    v_proj: torch.Tensor,
    gating_query: torch.Tensor,
    head: int,
    use_flash_attention: bool = False,  # unused, as in the reference
    BLK_SZ: int = 128,
    FLASH_SZ: int = 1024,                # unused, as in the reference
) -> torch.Tensor:
    """Diffusion-transformer self-attention on one token sequence:
        q = x . Wq + q_bias;  k, v, g = x . Wk, Wv, Wg;  out = softmax(q k^T K^-1/2 + bias, mask) v * sigmoid(g)
    pair (x) [N, C]; mask [N]; bias [head, N, N]; q_bias [C] (or [head, C/head]); weights as in
    _attention_cpp.  Returns [N, C].

    Beyond the reference (which takes one sequence per call, src/csrc/dot_product_attention.cpp:380-543): pair may be
    [S, N, C] -- S diffusion samples of the same tokens, mask [N] or [S, N] -- and the S samples then go through ONE
    projection GEMM and ONE attention launch in which they share every bias tile (the pair bias, the largest operand,
    is streamed once instead of S times).  Returns [S, N, C]."""
    ops._require_device(pair, mask, bias, q_proj, q_bias, k_proj, v_proj, gating_query)
    if pair.dim() == 3:
        S, N, C = pair.shape
        _check_weights(C, head, (q_proj, k_proj, v_proj, gating_query))
        if ops._DTYPE_CODE.get(pair.dtype) not in (ops.AF3_F32, ops.AF3_BF16):
            raise ValueError(f"unsupported dtype {pair.dtype}: float32 or bfloat16")
        y = _project(pair.reshape(S * N, C), (q_proj, k_proj, v_proj, gating_query), q_bias, head)
        return _attend(y, S, N, head, mask, bias)
    if pair.dim() != 2:
        raise ValueError(f"pair must be [N, C] or [S, N, C], got {tuple(pair.shape)}")
    N, C = pair.shape
    _check_weights(C, head, (q_proj, k_proj, v_proj, gating_query))
    dtype = pair.dtype
    code = ops._DTYPE_CODE.get(dtype)
    if code not in (ops.AF3_F32, ops.AF3_BF16):
        raise ValueError(f"unsupported dtype {dtype}: float32 or bfloat16")
    y = _project(pair, (q_proj, k_proj, v_proj, gating_query), q_bias, head)
    return _attend(y, 1, N, head, mask, bias).view(N, C)


def layernorm_pair_bias(pair: torch.Tensor, ln_weight: torch.Tensor, ln_bias: torch.Tensor, eps: float, proj_weight: torch.Tensor):
    """act_norm + pair_bias_projection + permute(2, 0, 1) of the reference module (src/af3_kernels/Attention.py:51-52) in
    one pass over the pair tensor: returns (normed [N1, N2, C], bias [head, N1, N2]).  One HIP kernel: a specialised one
    for bfloat16 pairs with 128 channels and 4 heads (the pair tensor's own shape), one wavefront per token for any other
    channel and head count (C <= 2048) in bfloat16 or float32.  Parameters in another dtype are cast to the pair's."""
    ops._require_device(pair, ln_weight, ln_bias, proj_weight)
    if pair.dim() != 3 or proj_weight.dim() != 2 or proj_weight.shape[1] != pair.shape[-1] or ln_weight.numel() != pair.shape[-1] or ln_bias.numel() != pair.shape[-1]:
        raise ValueError(f"pair must be [N1, N2, C] with ln_weight, ln_bias [C] and proj_weight [head, C], got {tuple(pair.shape)}, {tuple(ln_weight.shape)}, "
                         f"{tuple(ln_bias.shape)}, {tuple(proj_weight.shape)}")
    if pair.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"unsupported dtype {pair.dtype}: float32 or bfloat16")
    head, C = proj_weight.shape
    if C > 2048 or head > 64 or (2 + head) * C * 4 > 160 * 1024 - 1024:
        raise ValueError(f"layernorm_pair_bias takes at most 2048 channels and (2 + head) * C * 4 bytes of LDS, got C={C}, head={head}")
    ln_weight, ln_bias, proj_weight = [t.to(pair.dtype).contiguous() for t in (ln_weight, ln_bias, proj_weight)]
    if pair.stride(2) != 1:
        pair = pair.contiguous()
    if pair.numel() == 0:
        return torch.empty_like(pair), torch.empty(head, *pair.shape[:2], dtype=pair.dtype, device=pair.device)
    n_i, n_j = pair.shape[:2]
    normed = torch.empty(n_i, n_j, C, dtype=pair.dtype, device=pair.device)
    bias = torch.empty(head, n_i, n_j, dtype=pair.dtype, device=pair.device)
    arr = ctypes.c_int64 * 2
    with ops._on_device(pair.device):
        _lib.check(_lib.load().af3_layernorm_pair_bias(pair.data_ptr(), arr(pair.stride(0), pair.stride(1)), ln_weight.data_ptr(), ln_bias.data_ptr(),
                                                       float(eps), proj_weight.data_ptr(), normed.data_ptr(), bias.data_ptr(), arr(n_i * n_j, n_j), n_i, n_j, C, head,
                                                       ops._DTYPE_CODE[pair.dtype], ops._stream_ptr(pair.device)), "af3_layernorm_pair_bias")
    return normed, bias


class GridSelfAttentionCpp(torch.nn.Module):
    """Same constructor, parameters and forward as the reference module (src/af3_kernels/Attention.py:23-82):
    LayerNorm and the pair-bias projection are one kernel (layernorm_pair_bias), the rest is _attention_cpp."""

    def __init__(self, c_pair: int = 128, num_head: int = 4, transpose: bool = False):
        super().__init__()
        self.c_pair = c_pair
        self.num_head = num_head
        self.qkv_dim = self.c_pair // self.num_head
        self.transpose = transpose
        self.act_norm = torch.nn.LayerNorm(self.c_pair)
        self.pair_bias_projection = torch.nn.Linear(self.c_pair, self.num_head, bias=False)
        self.q_projection = torch.nn.Linear(self.c_pair, self.c_pair, bias=False)
        self.k_projection = torch.nn.Linear(self.c_pair, self.c_pair, bias=False)
        self.v_projection = torch.nn.Linear(self.c_pair, self.c_pair, bias=False)
        self.gating_query = torch.nn.Linear(self.c_pair, self.c_pair, bias=False)
        self.output_projection = torch.nn.Linear(self.c_pair, self.c_pair, bias=False)
        self.first_run = True
        self.q_proj = self.k_proj = self.v_proj = self.gq = self.out_proj = None

    def _pack(self, linear: torch.nn.Linear) -> torch.Tensor:
        w_t = linear.weight.T.contiguous()
        if w_t.dtype == torch.bfloat16:
            return ops.vnni_repack_tensor(w_t, 2, self.qkv_dim)
        # float32: one [C, K] panel per head (pair size 1), the layout _attention_impl<float> indexes
        return w_t.view(self.c_pair, self.num_head, self.qkv_dim).permute(1, 0, 2).contiguous().view(self.c_pair, self.c_pair)

    def _packed_weights(self):
        """Packed once, on the first forward, like the reference (weights are frozen for inference)."""
        if self.first_run:
            self.q_proj, self.k_proj, self.v_proj, self.gq = (
                self._pack(m) for m in (self.q_projection, self.k_projection, self.v_projection, self.gating_query))
            self.out_proj = self.output_projection.weight.T.contiguous()
            self.first_run = False
        return self.q_proj, self.k_proj, self.v_proj, self.gq, self.out_proj

    def forward(self, pair: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
        normed, bias = layernorm_pair_bias(pair, self.act_norm.weight, self.act_norm.bias, self.act_norm.eps, self.pair_bias_projection.weight)  # bias [head, N, N]
        rows = normed.transpose(0, 1) if self.transpose else normed         # attend along columns when transposed
        out = _attention_cpp(rows, mask, bias, *self._packed_weights(), self.num_head, False, 128 if pair.shape[1] > 256 else 64, 0)
        return out.transpose(0, 1) if self.transpose else out


def _narrow_linear_ok(x2: torch.Tensor, n_out: int) -> bool:
    """Shapes for which af3_linear beats the library GEMM (measured): bfloat16, 64 or 128 input channels, at most 128 outputs."""
    return (x2.dtype == torch.bfloat16 and x2.shape[1] in (64, 128) and n_out % 32 == 0 and n_out <= 128 and x2.shape[0] > 0 and x2.is_contiguous()
            and x2.data_ptr() % 16 == 0)


def _linear_rows(x2: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """x2 [M, K] . weight^T for weight [N, K] (nn.Linear layout) through af3_linear; the caller has checked the shape limits."""
    out = torch.empty(x2.shape[0], weight.shape[0], dtype=x2.dtype, device=x2.device)
    with ops._on_device(x2.device):
        _lib.check(_lib.load().af3_linear(x2.data_ptr(), weight.data_ptr(), out.data_ptr(), x2.shape[0], x2.shape[1], weight.shape[0], ops._DTYPE_CODE[x2.dtype],
                                          ops._stream_ptr(x2.device)), "af3_linear")
    return out


def _plain_weight(weight: torch.Tensor, vnni_repacked: bool, N_BLK: int) -> torch.Tensor:
    """[K, N] weight as the reference's callers hand it over -- plain, or VNNI panels of width N_BLK
    (vnni_repack_tensor(W, 2, N_BLK): [N/N_BLK][K/2][N_BLK][2]) -- back to plain [K, N]."""
    if not vnni_repacked:
        return weight
    K, N = weight.shape
    blk = min(N_BLK, N) if N_BLK > 0 else N
    if weight.dtype != torch.bfloat16 or N % blk != 0 or K % 2 != 0:
        raise ValueError("a VNNI-repacked weight is bfloat16 [K, N] with K even and N a multiple of N_BLK")
    return weight.reshape(N // blk, K // 2, blk, 2).permute(1, 3, 0, 2).reshape(K, N)


def gated_linear_unit_cpp(x: torch.Tensor, weight: torch.Tensor, vnni_repacked: bool = False, M_BLK: int = 128, N_BLK: int = 128) -> torch.Tensor:
    """silu(x @ W[:, :N]) * (x @ W[:, N:]) -- drop-in for the reference's gated_linear_unit_cpp (src/af3_kernels/__init__.py:
    21-28; src/csrc/gated_linear_unit.cpp:20-80).  x [..., K], weight [K, 2N] (plain or VNNI-repacked with N_BLK); returns
    [..., N] in x's dtype.  bfloat16 with K = 64 or 128 and N % 32 == 0 is one HIP kernel (the [.., 2N] product is never
    stored); other shapes (bfloat16 or float32) are a library GEMM for x @ W followed by the silu-and-multiply kernel
    (af3_silu_mul).  M_BLK and N_BLK are CPU blocking sizes (N_BLK also names the panel width of a repacked weight) and
    change nothing else."""
    ops._require_device(x, weight)
    if weight.dim() != 2 or weight.shape[0] != x.shape[-1] or weight.shape[1] % 2 != 0:
        raise ValueError(f"weight must be [K, 2N] with K = x.shape[-1] = {x.shape[-1]}, got {tuple(weight.shape)}")
    K, N = weight.shape[0], weight.shape[1] // 2
    lead = x.shape[:-1]
    if x.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"unsupported dtype {x.dtype}: float32 or bfloat16")
    if x.numel() == 0:
        return torch.empty(*lead, N, dtype=x.dtype, device=x.device)
    if not (x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and K in (64, 128) and N % 32 == 0):
        w = _cached((weight,), (bool(vnni_repacked), N_BLK, x.dtype, "glu_plain"), lambda: _plain_weight(weight, vnni_repacked, N_BLK).to(x.dtype).contiguous())
        y = torch.matmul(x.reshape(-1, K), w)                       # [M, 2N]: the library GEMM (hipBLASLt)
        out = torch.empty(y.shape[0], N, dtype=x.dtype, device=x.device)
        with ops._on_device(x.device):
            _lib.check(_lib.load().af3_silu_mul(y.data_ptr(), out.data_ptr(), y.shape[0], N, ops._DTYPE_CODE[x.dtype], ops._stream_ptr(x.device)), "af3_silu_mul")
        return out.view(*lead, N)
    wt = _cached((weight,), (bool(vnni_repacked), N_BLK, "glu"), lambda: _plain_weight(weight, vnni_repacked, N_BLK).t().contiguous())
    x2 = x.reshape(-1, K)
    if not x2.is_contiguous() or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    out = torch.empty(x2.shape[0], N, dtype=x.dtype, device=x.device)
    with ops._on_device(x.device):
        _lib.check(_lib.load().af3_gated_linear_unit(x2.data_ptr(), wt.data_ptr(), out.data_ptr(), x2.shape[0], K, N, ops._DTYPE_CODE[x.dtype],
                                                     ops._stream_ptr(x.device)), "af3_gated_linear_unit")
    return out.view(*lead, N)


class Linear(torch.nn.Module):
    """Bias-free linear layer with the reference's constructor (src/af3_kernels/__init__.py:138-163).  The reference repacks
    the weight into VNNI panels for its CPU GEMM; here the product runs on the plain weight: af3_linear for narrow layers
    (64 or 128 inputs, at most 128 outputs, bfloat16), a library GEMM (hipBLASLt) otherwise."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None, M_BLK: int = 128, N_BLK: int = 128) -> None:
        super().__init__()
        assert bias is False
        self.in_features, self.out_features = in_features, out_features
        self.weight = torch.nn.Parameter(torch.empty((out_features, in_features), device=device, dtype=dtype))
        self.register_parameter("bias", None)
        self.M_BLK, self.N_BLK = M_BLK, N_BLK

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        ops._require_device(input, self.weight)
        x2 = input.reshape(-1, self.in_features)
        if self.weight.dtype == input.dtype and self.weight.is_contiguous() and _narrow_linear_ok(x2, self.out_features):
            return _linear_rows(x2, self.weight).view(*input.shape[:-1], self.out_features)
        return torch.nn.functional.linear(input, self.weight)
