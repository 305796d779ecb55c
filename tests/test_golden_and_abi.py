"""CPU-only checks: the oracle against the committed golden vectors, the C-ABI library's
exported symbols and host-side validation (no kernel is launched here), and the host logic of
the Python wrapper."""
import ctypes
import glob
import os
import re

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "cfg*.npz")) + glob.glob(os.path.join(ROOT, "tests", "golden", "edge_*.npz")))   # the attention core's vectors


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_reproduces_golden(oracle, path):
    g = np.load(path)
    got = oracle.dpa_formula(g["q"], g["k"], g["v"], g["mask"], g["bias"])
    assert np.abs(got - g["expected"]).max() < 2e-6
    ref = oracle.dpa_reference(g["q"], g["k"], g["v"], g["mask"], g["bias"], BLK_SZ=64 if g["q"].shape[2] % 64 == 0 else 128)
    # the compiled reference dilutes an all-dropped row with its zero padding when L % BLK != 0 (tools.cpp pads V with 0,
    # dot_product_attention.cpp:54 pads the mask with 1.0); everywhere else it agrees with the formula
    B, L = g["q"].shape[0], g["q"].shape[2]
    keep = np.broadcast_to(g["mask"].reshape(-1, L), (B, L)) if g["mask"].ndim == 1 else g["mask"]
    rows = keep.any(1)
    assert np.abs(ref[rows] - g["expected"][rows]).max() < 2e-5


def test_oracle_reproduces_the_fused_callers_golden_vectors(oracle):
    """The C oracle against the vectors tests/golden/make_golden.py wrote from the independent float64 numpy forms
    (oracle/dpa_numpy.py): grid and diffusion self-attention, LayerNorm + pair bias, gated linear unit."""
    gdir = os.path.join(ROOT, "tests", "golden")
    g = np.load(os.path.join(gdir, "grid_attention_B3_N40_C128.npz"))
    got = oracle.fused_attention_formula(g["x"], g["mask"], g["bias"], g["wq"], g["wk"], g["wv"], g["wg"], g["wo"], None, head=int(g["head"]))
    assert np.abs(got - g["expected"]).max() < 3e-6
    g = np.load(os.path.join(gdir, "self_attention_N50_C96.npz"))
    got = oracle.fused_attention_formula(g["x"], g["mask"], g["bias"], g["wq"], g["wk"], g["wv"], g["wg"], None, g["q_bias"], head=int(g["head"]))
    assert got.shape == (50, 96) and np.abs(got - g["expected"]).max() < 3e-6
    g = np.load(os.path.join(gdir, "layernorm_pair_bias_6x9x128.npz"))
    normed, bias = oracle.layernorm_pair_bias(g["pair"], g["gamma"], g["beta"], g["wb"], float(g["eps"]))
    assert np.abs(normed - g["normed"]).max() < 3e-6 and np.abs(bias - g["bias"]).max() < 3e-6
    g = np.load(os.path.join(gdir, "glu_70x128_N64.npz"))
    assert np.abs(oracle.gated_linear_unit(g["x"], g["weight"]) - g["expected"]).max() < 1e-5


def test_golden_cfg1_is_the_named_case():
    from af3_kernels_amd.synthetic import CASES, make_inputs
    g = np.load(os.path.join(ROOT, "tests", "golden", "cfg1_fp32.npz"))
    q, k, v, mask, bias = make_inputs(CASES["cfg1"])
    assert q.shape == (2, 4, 128, 32) and bias.shape == (4, 128, 128) and mask.shape == (2, 128)
    assert mask[0].all() and mask[1, :112].all() and not mask[1, 112:].any()
    assert np.array_equal(q.numpy(), g["q"]) and np.array_equal(bias.numpy(), g["bias"])


# ---- the C-ABI library ---------------------------------------------------------------------

def declared_symbols():
    text = open(os.path.join(ROOT, "include", "af3_dpa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(af3_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from af3_kernels_amd import _lib
    lib = _lib.load()
    names = declared_symbols()
    assert "af3_dpa_forward" in names and len(names) >= 8
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/af3_dpa.h but not exported"
    assert sorted(_lib.SYMBOLS) == names
    assert lib.af3_abi_version() == _lib.ABI_VERSION
    assert lib.af3_status_string(0) == b"ok"


def test_params_struct_matches_header_layout():
    from af3_kernels_amd._lib import DpaParams
    # 6 pointers, 4 dims, 4*3 + 2 + 1 strides (int64), 4 int32, 4 floats, 2 int32, 2 pointers, 1 int64, 2 pointers
    assert ctypes.sizeof(DpaParams) == 6 * 8 + 4 * 8 + 15 * 8 + 4 * 4 + 4 * 4 + 2 * 4 + 8 + 8 + 8 + 8 + 8 + 8 + 3 * 8
    assert DpaParams.gate.offset == ctypes.sizeof(DpaParams) - 32 and DpaParams.k_lo.offset == DpaParams.gate.offset - 8


def _params(**kw):
    from af3_kernels_amd._lib import DpaParams, AF3_BF16
    p = DpaParams()
    B, H, L, D = 2, 4, 64, 32
    p.B, p.H, p.L, p.D = B, H, L, D
    for name in ("q", "k", "v", "out"):
        setattr(p, name, 0x1000)   # never dereferenced: validation fails first or select_kernel is host-only
        setattr(p, name + "_stride", (ctypes.c_int64 * 3)(H * L * D, L * D, D))
    p.io_dtype = p.out_dtype = p.mma_dtype = p.bias_dtype = AF3_BF16
    p.softmax_scale = D ** -0.5
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def test_host_validation_returns_error_codes_instead_of_exiting():
    from af3_kernels_amd import _lib
    lib = _lib.load()
    fwd = lib.af3_dpa_forward
    assert fwd(None, None) == -1
    assert fwd(ctypes.byref(_params(q=None)), None) == -1
    assert fwd(ctypes.byref(_params(L=0)), None) == -3
    assert fwd(ctypes.byref(_params(D=256)), None) == -5
    assert fwd(ctypes.byref(_params(io_dtype=7)), None) == -2
    assert fwd(ctypes.byref(_params(io_dtype=0)), None) == -2            # fp32 storage with bf16 arithmetic
    assert fwd(ctypes.byref(_params(q_stride=(ctypes.c_int64 * 3)(1, 1, 8))), None) == -4   # rows overlap
    assert fwd(ctypes.byref(_params(softmax_scale=0.0)), None) == -7
    assert fwd(ctypes.byref(_params(bias=0x1000, bias_stride=(ctypes.c_int64 * 2)(64 * 64, 8))), None) == -4
    for code in range(-8, 1):
        assert lib.af3_status_string(code) != b"unknown status"
    with pytest.raises(ValueError):
        _lib.check(-3, "x")
    with pytest.raises(RuntimeError):
        _lib.check(-6, "x")


def test_kernel_selection_is_host_only_and_follows_alignment():
    from af3_kernels_amd import _lib
    sel = _lib.load().af3_dpa_select_kernel
    assert sel(ctypes.byref(_params())) == 1                              # bf16 MFMA
    assert sel(ctypes.byref(_params(force_generic=1))) == 0
    assert sel(ctypes.byref(_params(mma_dtype=0))) == 0                   # bf16 storage, fp32 arithmetic
    assert sel(ctypes.byref(_params(q=0x1002))) == 0                      # misaligned rows -> fp32-FMA kernel
    assert sel(ctypes.byref(_params(D=20))) == 0                          # head_dim not a multiple of 8
    s96 = (ctypes.c_int64 * 3)(4 * 64 * 96, 64 * 96, 96)
    assert sel(ctypes.byref(_params(D=96, q_stride=s96, k_stride=s96, v_stride=s96, out_stride=s96))) == 0   # head_dim > 64
    assert sel(ctypes.byref(_params(D=96))) == -4                         # rows of 96 with stride 32 overlap
    assert sel(ctypes.byref(_params(io_dtype=0, mma_dtype=0, out_dtype=0, bias_dtype=0))) == 3   # fp32 storage -> fp32 MFMA
    assert sel(ctypes.byref(_params(io_dtype=0, mma_dtype=0, out_dtype=0, bias_dtype=0, k=0x2004))) == 0   # rows not 16-byte aligned
    assert sel(ctypes.byref(_params(io_dtype=0, mma_dtype=0, out_dtype=0, bias_dtype=0, force_generic=1))) == 0
    assert sel(ctypes.byref(_params(L=-1))) == -3


def test_elementwise_entry_points_validate_on_the_host():
    from af3_kernels_amd import _lib
    lib = _lib.load()
    assert lib.af3_convert(None, 0, None, 1, 0, None) == 0               # empty: nothing to do
    assert lib.af3_convert(None, 0, None, 1, 8, None) == -1
    assert lib.af3_convert(0x1000, 1, 0x2000, 2, 8, None) == -2          # bf16 -> fp8 goes through af3_quantize_fp8_e4m3
    assert lib.af3_amax(0x1000, 2, 8, 0x2000, None) == -2
    assert lib.af3_vnni_repack_bf16(0x1000, 0x2000, 16, 24, 7, None) == -7   # N % BLK_SZ != 0: the reference exits here
    assert lib.af3_vnni_repack_bf16(0x1000, 0x2000, 15, 24, 8, None) == -7
    arr = ctypes.c_int64 * 2
    assert lib.af3_pad_nd(0x1000, 0x2000, 2, arr(4, 4), arr(4, 1), arr(2, 8), 4, 0, None) == -3   # shrinking
    assert lib.af3_pad_nd(0x1000, 0x2000, 9, arr(4, 4), arr(4, 1), arr(4, 8), 4, 0, None) == -3
    assert lib.af3_quantize_fp8_e4m3(0x1000, 1, 0x2000, 8, 6, 6, 0, 0, 6, 1.0, 0x3000, None, None, None) == -7    # cols % 4
    qkv = lib.af3_quantize_qkv_fp8_e4m3
    good = dict(q=0x1000, k=0x2000, v=0x3000, sd=1, B=1, H=2, L=10, D=8, pre=1.0, q8=0x4000, k8=0x5000, v8t=0x6000, vs=16, qlo=None, klo=None, ds=0x7000, sc=0x8000)
    call = lambda **kw: qkv(*[{**good, **kw}[n] for n in ("q", "k", "v", "sd", "B", "H", "L", "D", "pre", "q8", "k8", "v8t", "vs", "qlo", "klo", "ds", "sc")], None)
    assert call(D=6) == -7            # head_dim % 4
    assert call(vs=8) == -4           # transposed rows shorter than L
    assert call(vs=14) == -4          # not a multiple of 4
    assert call(sd=2) == -2           # fp8 source
    assert call(sc=None) == -1
    assert call(L=0) == -3


def test_wrapper_rejects_cpu_tensors_and_bad_shapes():
    import af3_kernels_amd as af3
    q = torch.randn(1, 2, 16, 8)
    mask = torch.ones(16, dtype=torch.bool)
    bias = torch.zeros(2, 16, 16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        af3.dot_product_attention_cpp(q, q, q, mask, bias)
    with pytest.raises(ValueError):
        af3.dot_product_attention_cpp(q.to(torch.float16), q, q, mask, bias)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        af3.vnni_repack_tensor(torch.zeros(4, 4, dtype=torch.bfloat16))


def test_wrapper_signature_matches_the_reference():
    import inspect
    import af3_kernels_amd as af3
    sig = inspect.signature(af3.dot_product_attention_cpp)
    assert list(sig.parameters) == ["q", "k", "v", "mask", "bias", "use_flash_attention", "BLK_SZ", "FLASH_SZ"]
    assert [sig.parameters[n].default for n in ("use_flash_attention", "BLK_SZ", "FLASH_SZ")] == [False, 128, 1024]
    assert list(inspect.signature(af3.pad_and_align_tensor).parameters) == ["x", "shape", "need_init", "init", "alignment"]
    assert list(inspect.signature(af3.vnni_repack_tensor).parameters) == ["x", "type", "BLK_SZ"]
    assert list(inspect.signature(af3.print_debug_timers).parameters) == ["tid", "detailed"]
    assert hasattr(torch.ops.af3_kernels, "dot_product_attention") and hasattr(torch.ops.af3_kernels, "dpa_forward")


def test_mask_lifting_follows_the_reference_wrapper():
    from af3_kernels_amd.ops import _lift_mask
    m1 = torch.tensor([1, 0, 1, 1], dtype=torch.bool)
    assert _lift_mask(m1, 4).shape == (1, 4) and _lift_mask(m1, 4).dtype == torch.uint8
    m2 = torch.tensor([[1.0, 0.0, 2.0, 0.0]])
    assert _lift_mask(m2, 4).tolist() == [[1, 0, 1, 0]]                  # truthy = attend
    m4 = torch.ones(3, 1, 1, 4, dtype=torch.bool)
    assert _lift_mask(m4, 4).shape == (3, 4)
    assert _lift_mask(m1, 4).data_ptr() == m1.data_ptr()                 # bool masks are reinterpreted, not copied


def test_struct_mirrors_match_what_a_c_compiler_lays_out(tmp_path):
    """sizeof / offsetof of both parameter structs as gcc sees include/af3_dpa.h, against the ctypes mirrors."""
    import shutil
    import subprocess
    from af3_kernels_amd._lib import DpaParams, GridAttentionParams
    if shutil.which("gcc") is None:
        pytest.skip("no C compiler")
    fields = {"af3_dpa_params": (DpaParams, ["q", "B", "q_stride", "bias_stride", "io_dtype", "softmax_scale", "force_generic", "device_descales", "workspace", "q_lo", "gate", "gate_stride"]),
              "af3_grid_attention_params": (GridAttentionParams, ["pair", "pair_stride", "q_proj", "gating_query", "bias", "bias_stride", "bias_dtype", "dtype", "key_mask", "key_mask_stride_b",
                                                                 "out", "out_stride", "B", "head", "workspace", "workspace_bytes"])}
    lines = ["#include <stdio.h>", "#include <stddef.h>", '#include "af3_dpa.h"', "int main(void) {"]
    for sname, (_, names) in fields.items():
        lines.append(f'printf("{sname} %zu\\n", sizeof({sname}));')
        lines += [f'printf("{sname}.{n} %zu\\n", offsetof({sname}, {n}));' for n in names]
    lines += ["return 0; }"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    got = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for sname, (cls, names) in fields.items():
        assert int(got[sname]) == ctypes.sizeof(cls)
        for n in names:
            assert int(got[f"{sname}.{n}"]) == getattr(cls, n).offset, (sname, n)


def _grid_params(**kw):
    from af3_kernels_amd._lib import GridAttentionParams, AF3_BF16
    g = GridAttentionParams()
    B, N, C = 64, 256, 128
    g.pair = g.out = g.q_proj = g.k_proj = g.v_proj = g.gating_query = 0x1000   # never dereferenced on the host
    g.pair_stride = g.out_stride = (ctypes.c_int64 * 2)(N * C, C)
    g.B, g.N, g.C, g.head = B, N, C, 4
    g.dtype = g.bias_dtype = AF3_BF16
    for k, v in kw.items():
        setattr(g, k, v)
    return g


def test_grid_attention_entry_points_validate_on_the_host():
    from af3_kernels_amd import _lib
    lib = _lib.load()
    sup, ws, fwd = lib.af3_grid_attention_supported, lib.af3_grid_attention_workspace_bytes, lib.af3_grid_attention_forward
    assert sup(ctypes.byref(_grid_params())) == 1
    assert ws(ctypes.byref(_grid_params())) == 0                                       # no bias, no workspace
    nb = (ctypes.c_int64 * 2)(256 * 256, 256)
    assert ws(ctypes.byref(_grid_params(bias=0x1000, bias_stride=nb))) == 4 * 8 * 4 * 4096   # heads x query blocks x key tiles x 4 KB
    assert sup(ctypes.byref(_grid_params(C=256))) == 0 and sup(ctypes.byref(_grid_params(head=8))) == 0
    assert sup(ctypes.byref(_grid_params(dtype=0))) == 0                               # float32 rows: composed by the caller
    assert sup(ctypes.byref(_grid_params(N=1100, pair_stride=(ctypes.c_int64 * 2)(1100 * 128, 128), out_stride=(ctypes.c_int64 * 2)(1100 * 128, 128)))) == 0   # K and V no longer fit in LDS
    assert sup(ctypes.byref(_grid_params(pair=0x1004))) == 0                           # rows not 16-byte aligned
    assert fwd(None, None) == -1
    assert fwd(ctypes.byref(_grid_params(q_proj=None)), None) == -1
    assert fwd(ctypes.byref(_grid_params(N=0)), None) == -3
    assert fwd(ctypes.byref(_grid_params(head=3)), None) == -3                         # 128 channels do not split into 3 heads
    assert fwd(ctypes.byref(_grid_params(pair_stride=(ctypes.c_int64 * 2)(256 * 128, 64))), None) == -4
    assert fwd(ctypes.byref(_grid_params(C=256, pair_stride=(ctypes.c_int64 * 2)(256 * 256, 256), out_stride=(ctypes.c_int64 * 2)(256 * 256, 256))), None) == -7   # valid but unsupported
    assert fwd(ctypes.byref(_grid_params(bias=0x1000, bias_stride=nb)), None) == -7    # a bias needs the workspace


def test_fused_wrappers_match_the_reference_signatures():
    import inspect
    import af3_kernels_amd as af3
    sig = inspect.signature(af3._attention_cpp)
    assert list(sig.parameters) == ["pair", "mask", "bias", "q_proj", "k_proj", "v_proj", "gating_query", "out_proj", "head", "use_flash_attention", "BLK_SZ", "FLASH_SZ"]
    assert [sig.parameters[n].default for n in ("use_flash_attention", "BLK_SZ", "FLASH_SZ")] == [False, 128, 1024]
    sig = inspect.signature(af3.self_attention_cpp)
    assert list(sig.parameters) == ["pair", "mask", "bias", "q_proj", "q_bias", "k_proj", "v_proj", "gating_query", "head", "use_flash_attention", "BLK_SZ", "FLASH_SZ"]
    mod = af3.GridSelfAttentionCpp(64, 2, transpose=True)
    assert sorted(dict(mod.named_parameters())) == sorted(
        ["act_norm.weight", "act_norm.bias", "pair_bias_projection.weight", "q_projection.weight", "k_projection.weight", "v_projection.weight",
         "gating_query.weight", "output_projection.weight"])
    x = torch.randn(2, 8, 64)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        af3._attention_cpp(x, torch.ones(2, 8, dtype=torch.bool), torch.zeros(2, 8, 8), *([torch.zeros(64, 64)] * 5), 2)


def test_weight_unpacking_inverts_the_panel_layout(oracle):
    """fused._unpack_panels undoes vnni_repack_tensor(W_t, 2, K) (checked against the oracle's repack) and the float32 panels."""
    from af3_kernels_amd import fused
    C, head = 64, 4
    K = C // head
    g = torch.Generator().manual_seed(2)
    w = torch.randn(C, C, generator=g).to(torch.bfloat16)
    packed = torch.from_numpy(oracle.vnni_repack(w.view(torch.int16).numpy().view(np.uint16), K).view(np.int16)).view(torch.bfloat16)
    assert torch.equal(fused._unpack_panels(packed, head), w)
    wf = torch.randn(C, C, generator=g)
    panels = wf.view(C, head, K).permute(1, 0, 2).contiguous().view(C, C)
    assert torch.equal(fused._unpack_panels(panels, head), wf)


def test_row_op_entry_points_validate_on_the_host():
    """af3_gated_linear_unit, af3_linear, af3_silu_mul and af3_layernorm_pair_bias refuse malformed calls with a status code, before any launch."""
    from af3_kernels_amd import _lib
    lib = _lib.load()
    P, BF, F32 = 0x1000, _lib.AF3_BF16, _lib.AF3_F32
    for fn in (lib.af3_gated_linear_unit, lib.af3_linear):
        assert fn(None, P, P, 64, 128, 64, BF, None) == -1
        assert fn(P, P, P, 0, 128, 64, BF, None) == -3
        assert fn(P, P, P, 64, 128, 64, F32, None) == -2                  # bfloat16 only
        assert fn(P, P, P, 64, 96, 64, BF, None) == -7                    # 64 or 128 input channels
        assert fn(P, P, P, 64, 128, 48, BF, None) == -7                   # outputs in tiles of 32 columns
        assert fn(P + 2, P, P, 64, 128, 64, BF, None) == -7               # rows not 16-byte aligned
    ln = lib.af3_layernorm_pair_bias
    ps, bs = (ctypes.c_int64 * 2)(9 * 128, 128), (ctypes.c_int64 * 2)(6 * 9, 9)
    assert ln(None, ps, P, P, 1e-5, P, P, P, bs, 6, 9, 128, 4, BF, None) == -1
    assert ln(P, ps, P, P, 1e-5, P, P, P, bs, 0, 9, 128, 4, BF, None) == -3
    assert ln(P, ps, P, P, 1e-5, P, P, P, bs, 6, 9, 128, 4, _lib.AF3_FP8_E4M3, None) == -2   # bfloat16 or float32
    assert ln(P, ps, P, P, 1e-5, P, P, P, bs, 6, 9, 0, 4, BF, None) == -3
    assert ln(P, (ctypes.c_int64 * 2)(9 * 4096, 4096), P, P, 1e-5, P, P, P, bs, 6, 9, 4096, 4, BF, None) == -7   # at most 2048 channels
    assert ln(P, (ctypes.c_int64 * 2)(9 * 1024, 1024), P, P, 1e-5, P, P, P, bs, 6, 9, 1024, 64, BF, None) == -7  # gamma, beta and the weights must fit in LDS
    assert ln(P + 1, ps, P, P, 1e-5, P, P, P, bs, 6, 9, 128, 4, BF, None) == -7                                     # not aligned to the element size
    assert ln(P, (ctypes.c_int64 * 2)(9 * 128, 64), P, P, 1e-5, P, P, P, bs, 6, 9, 128, 4, BF, None) == -4   # tokens overlap
    assert ln(P, ps, P, P, 1e-5, P, P, P, (ctypes.c_int64 * 2)(6 * 9, 4), 6, 9, 128, 4, BF, None) == -4        # bias rows overlap
    assert ln(P, ps, P, P, -1.0, P, P, P, bs, 6, 9, 128, 4, BF, None) == -7
    sm = lib.af3_silu_mul
    assert sm(None, P, 4, 8, BF, None) == -1 and sm(P, P, 0, 8, BF, None) == -3 and sm(P, P, 4, 8, _lib.AF3_FP8_E4M3, None) == -2


def test_derived_weight_cache_follows_tensor_identity_and_version():
    """The cache of matrices derived from weights (host logic of the fused callers): same live tensor and version ->
    same object; an in-place update or another tensor at a recycled id -> recomputed; entries of dead weights go."""
    import gc
    import torch
    from af3_kernels_amd import fused
    fused._W_CACHE.clear()
    calls = []

    def derive(t):
        return fused._cached((t,), ("unit",), lambda: calls.append(1) or t.clone())

    w = torch.arange(6.0)
    a = derive(w)
    assert derive(w) is a and len(calls) == 1
    w.add_(1.0)                                  # bumps the version
    b = derive(w)
    assert b is not a and len(calls) == 2 and torch.equal(b, w)
    other = torch.arange(6.0)
    assert derive(other) is not b and len(calls) == 3
    n_before = len(fused._W_CACHE)
    del w, other
    gc.collect()
    derive(torch.zeros(3))                       # an insertion purges what belonged to tensors that no longer exist
    assert len(fused._W_CACHE) == n_before - 2 + 1
    # a stale entry under a recycled id must not be served: forge one
    t = torch.ones(2)
    key = (id(t), "unit")
    dead = torch.ones(1)
    import weakref
    fused._W_CACHE[key] = ((weakref.ref(dead),), (dead._version,), "stale")
    got = derive(t)
    assert not isinstance(got, str) and torch.equal(got, t)
    # a tensor whose storage was swapped under the same object and version (set_) is seen through its address
    u = torch.arange(4.0)
    first = derive(u)
    u.set_(torch.arange(4.0) + 10.0)
    second = derive(u)
    assert second is not first and torch.equal(second, u)
    # a write that bypasses the version counter cannot be seen; clear_weight_cache() is the documented remedy
    n = len(calls)
    u.data.copy_(torch.zeros(4))
    assert derive(u) is second and len(calls) == n
    fused.clear_weight_cache()
    third = derive(u)
    assert len(calls) == n + 1 and torch.equal(third, torch.zeros(4))


def test_no_device_is_reported_as_such_before_anything_is_launched():
    """Without a gfx950 as the current device (this test runs where there is no GPU at all) a well-formed call
    returns AF3_ERR_NO_DEVICE_CODE from the host-side check; nothing is enqueued."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the arch check passes here")
    from af3_kernels_amd import _lib
    lib = _lib.load()
    assert lib.af3_dpa_forward(ctypes.byref(_params()), None) == -8
    with pytest.raises(RuntimeError, match="gfx950"):
        _lib.check(-8, "af3_dpa_forward")


def test_static_scratch_entry_point_rejects_calls_beyond_its_limit_on_the_host():
    """af3_dpa_forward_static_scratch: a call whose scratch need exceeds the library's built-in array returns
    AF3_ERR_SCRATCH_LIMIT before anything touches a device; malformed calls return the usual codes."""
    from af3_kernels_amd import _lib
    lib = _lib.load()
    fwd, need = lib.af3_dpa_forward_static_scratch, lib.af3_dpa_workspace_bytes
    assert fwd(None, None) == -1
    assert fwd(ctypes.byref(_params(L=0)), None) == -3
    L = 2048
    st = (ctypes.c_int64 * 3)(4 * L * 32, L * 32, 32)
    # (a bias whose rows are only 8-byte aligned: a call with so few batch rows would otherwise read it in place, without scratch)
    big = _params(B=2, H=4, L=L, bias=0x1008, bias_stride=(ctypes.c_int64 * 2)(L * L, L), q_stride=st, k_stride=st, v_stride=st, out_stride=st)
    assert need(ctypes.byref(big)) > _lib.STATIC_SCRATCH_BYTES
    assert fwd(ctypes.byref(big), None) == -9
    assert b"scratch" in lib.af3_status_string(-9)
    with pytest.raises(ValueError):
        _lib.check(-9, "x")


def test_workspace_query_follows_the_batch_size_at_which_a_bias_rewrite_pays_off():
    """af3_dpa_workspace_bytes (host only): a bf16 bias with 16-byte aligned rows is read in place -- no workspace -- while the
    batch has fewer rows than about 224 + 2.4e8 / (H L^2); beyond that, or when the rows cannot be staged, the fp32 rewrite
    (H * ceil(L/32)^2 blocks of 4 KB) is asked for."""
    from af3_kernels_amd import _lib
    lib = _lib.load()
    need = lib.af3_dpa_workspace_bytes

    def call(B, H, L, bias=0x1000, row_stride=None):
        st = (ctypes.c_int64 * 3)(H * L * 32, L * 32, 32)
        rs = L if row_stride is None else row_stride
        return need(ctypes.byref(_params(B=B, H=H, L=L, bias=bias, bias_stride=(ctypes.c_int64 * 2)(L * rs, rs), q_stride=st, k_stride=st, v_stride=st, out_stride=st)))

    rewrite = lambda H, L: H * ((L + 31) // 32) ** 2 * 4096
    assert call(384, 4, 384) == 0                        # cfg2: 384 < 224 + 2.4e8 / (4 * 384^2) = 637
    assert call(700, 4, 384) == rewrite(4, 384)
    assert call(300, 4, 768) == 0                        # 300 < 327
    assert call(768, 4, 768) == rewrite(4, 768)          # cfg4
    assert call(64, 16, 1536) == 0 and call(256, 16, 1536) == rewrite(16, 1536)   # 230 for the diffusion bias
    assert call(64, 4, 768, bias=0x1008) == rewrite(4, 768)          # rows only 8-byte aligned: not staged
    assert call(64, 4, 396) == rewrite(4, 396)                       # L % 8 != 0: not staged
    assert call(64, 4, 768, bias=None) == 0 and call(1, 16, 768) == 0


def test_argument_blocks_and_weight_cache_can_be_built_from_several_threads():
    """The Python side promises that calls may come from several threads: the per-layout templates of the argument block and
    the derived-weight cache are shared, filled on a miss and cleared when full.  Eight threads build blocks for more
    layouts than the template cache holds (so it is cleared under their feet) and look up derived weights of tensors
    that come and go; every block must describe exactly the tensors it was built for."""
    import threading
    from af3_kernels_amd import fused, ops, _lib
    errors = []

    def worker(seed):
        try:
            g = torch.Generator().manual_seed(seed)
            for i in range(300):
                B, H, L, D = 1 + (seed + i) % 5, 1 + i % 7, 8 * (1 + (i * 7 + seed) % 40), 8 * (1 + i % 4)
                q = torch.empty(B, H, L, D, dtype=torch.bfloat16)
                k, v, out = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
                bias = torch.empty(H, L, L, dtype=torch.bfloat16)
                keep = torch.ones(B, L, dtype=torch.uint8)
                p = ops._fill_params(q, k, v, keep, bias, out, _lib.AF3_BF16, False)
                assert (p.B, p.H, p.L, p.D) == (B, H, L, D)
                assert tuple(p.q_stride) == tuple(q.stride()[:3]) and tuple(p.bias_stride) == (L * L, L)
                assert p.q == q.data_ptr() and p.k == k.data_ptr() and p.v == v.data_ptr() and p.out == out.data_ptr()
                assert p.bias == bias.data_ptr() and p.key_mask == keep.data_ptr() and p.key_mask_stride_b == (0 if B == 1 else L)
                assert abs(p.softmax_scale - D ** -0.5) < 1e-7
                w = torch.randn(4 + i % 3, 5, generator=g)
                got = fused._cached((w,), ("t", seed % 2), lambda: w.t().contiguous())
                assert torch.equal(got, w.t())
                if i % 50 == 49:
                    fused.clear_weight_cache()
        except Exception as e:   # noqa: BLE001 -- reported by the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(s,)) for s in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors[:3]
    assert len(ops._PARAM_TEMPLATES) <= 256 and len(fused._W_CACHE) <= fused._W_CACHE_MAX


def test_traffic_digest_follows_the_code_and_not_its_commentary():
    """bench.py reports roofline.traffic from a committed counter summary only while the kernel sources' code has the digest the
    counters were collected with.  The digest ignores comments and whitespace (no hand re-stamping after an edit of the
    commentary), changes with any other edit, keeps string literals intact -- and every committed summary matches the
    sources as they are, so that a kernel change without fresh counters shows up here and not as a silent null."""
    import sys
    sys.path.insert(0, ROOT)
    import bench
    a = 'int x = 1; // one\n/* block\n comment */ asm volatile("s_nop 0 // kept\\n\\t" ::: "memory");  char c = \'"\';\n'
    b = 'int x=1;asm volatile("s_nop 0 // kept\\n\\t":::"memory");\n\n   char c=\'"\'; // trailing words\n'
    assert bench._code_only(a) == bench._code_only(b)
    assert bench._code_only(a) != bench._code_only(a.replace("x = 1", "x = 2"))
    assert bench._code_only(a) != bench._code_only(a.replace("// kept", "// changed"))     # inside a string literal: code
    digest = bench.kernel_sources_digest()
    for name, fname in bench.TRAFFIC_PROFILES.items():
        text = open(os.path.join(ROOT, "profiles", fname)).read()
        assert "kernel_code_sha256: " + digest in text, f"profiles/{fname} was collected with other kernel code: re-collect the counters"
        assert bench.measured_traffic_bytes(name) > 0
