"""GPU parity tests: the HIP kernels, called through the Python drop-in (which goes through the
C ABI of include/af3_dpa.h), against the CPU oracle on the same seeded inputs.

Tolerances are the ones the task states, max-abs against the fp64 formula evaluated on the
same (already rounded) inputs: 1e-4 for fp32, 2e-2 for bf16.  Cases too large for the oracle
are checked on sampled batch rows and through size-independent properties.
"""
import glob
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module")
def af3():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import af3_kernels_amd
    af3_kernels_amd._lib.load()   # raises if libaf3_dpa.so is missing: no fallback
    return af3_kernels_amd


def dev(*ts):
    return [t.cuda() if t is not None else None for t in ts]


def f32np(t):
    return t.detach().float().cpu().numpy()


def run_case(af3, oracle, q, k, v, mask, bias, tol=None, expect_kernel=None, **kw):
    """q,k,v,bias: CPU torch tensors (fp32 or bf16); returns the max-abs error vs the formula."""
    tol = TOL[q.dtype] if tol is None else tol
    dq, dk, dv, dm, db = dev(q, k, v, mask, bias)
    if expect_kernel is not None:
        assert af3.selected_kernel(dq, dk, dv, dm, db) == expect_kernel
    print(f"case B,H,L,D={tuple(q.shape)} dtype={q.dtype} mask={None if mask is None else tuple(mask.shape)}", flush=True)
    out = af3.dot_product_attention_cpp(dq, dk, dv, dm, db, **kw)
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == q.dtype and out.is_cuda
    assert out.data_ptr() != dq.data_ptr()
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), mask.numpy(), f32np(bias))
    got = f32np(out)
    assert np.isfinite(got).all()
    err = float(np.abs(got - want).max())
    assert err <= tol, f"max abs err {err} > {tol}"
    return err


def rand_inputs(B, H, L, D, dtype, seed=0, mask="none", mask_rank=2):
    g = torch.Generator().manual_seed(seed)
    q, k, v = [torch.randn(B, H, L, D, generator=g).to(dtype) for _ in range(3)]
    bias = torch.randn(H, L, L, generator=g).to(dtype)
    if mask == "none":
        m = torch.ones(B, L, dtype=torch.bool)
    elif mask == "random":
        m = torch.rand(B, L, generator=g) < 0.7
        m[:, 0] = True
    elif mask == "tail":
        m = torch.ones(B, L, dtype=torch.bool)
        m[:, L - max(1, L // 10):] = False
    if mask_rank == 1:
        m = m[0].clone()
    return q, k, v, m, bias


# ---- golden vectors -------------------------------------------------------------------------

GOLDEN = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "cfg*.npz")) + glob.glob(os.path.join(ROOT, "tests", "golden", "edge_*.npz")))   # the attention core's vectors


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_golden_vectors(af3, path, dtype):
    g = np.load(path)
    if dtype == torch.bfloat16 and "cfg1" in path:
        pytest.skip("cfg1 is the fp32 case (its inputs are not bf16-representable)")
    q, k, v, bias = [torch.from_numpy(g[n]).to(dtype).cuda() for n in ("q", "k", "v", "bias")]
    mask = torch.from_numpy(g["mask"]).cuda()
    out = af3.dot_product_attention_cpp(q, k, v, mask, bias)
    torch.cuda.synchronize()
    err = np.abs(f32np(out) - g["expected"]).max()
    assert err <= TOL[dtype], err


def test_cfg1_fp32_plumbing_case(af3, oracle):
    from af3_kernels_amd.synthetic import CASES, make_inputs
    q, k, v, mask, bias = make_inputs(CASES["cfg1"])
    err = run_case(af3, oracle, q, k, v, mask, bias, expect_kernel="fp32_mfma")
    assert err < 1e-5   # fp32 matrix cores with an fp32 softmax sit far inside the 1e-4 budget


# ---- bf16 matrix-core kernel ----------------------------------------------------------------

@pytest.mark.parametrize("B,H,L,D,mask,rank", [
    (2, 4, 128, 32, "none", 2),
    (3, 4, 384, 32, "tail", 2),      # triangle attention shape, tail padding
    (2, 4, 768, 32, "random", 2),    # headline shape, random mask
    (1, 16, 768, 24, "tail", 1),     # pair-biased single attention: head_dim 24, 1-D mask
    (2, 16, 128, 48, "random", 2),   # diffusion shape of the reference harness, head_dim 48
    (2, 2, 256, 64, "random", 2),
    (2, 2, 192, 16, "tail", 2),
    (3, 4, 37, 32, "random", 2),     # L = 37: the reference harness's small case (odd length)
    (2, 4, 65, 32, "none", 1),
    (1, 4, 1491, 32, "tail", 2),     # the reference harness's default length
    (1, 2, 1000, 24, "random", 1),
])
def test_bf16_mfma_matches_formula(af3, oracle, B, H, L, D, mask, rank):
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=L + D, mask=mask, mask_rank=rank)
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")


@pytest.mark.parametrize("B,H,L,D,live", [
    (1, 2, 300, 24, None),     # 20 query blocks, 5 key tiles: four wavefronts share a block, one gets two tiles
    (1, 2, 300, 32, 40),       # only the first tile is live: three of the four wavefronts have no tile at all
    (1, 4, 520, 32, (260, 330)),  # live keys in the middle: tiles 4 and 5 only
    (1, 2, 320, 64, None),     # head_dim 64: two wavefronts per block
    (2, 2, 100, 32, None),     # two key tiles, bias through the fragment-ordered workspace
    (1, 1, 2048, 32, None),    # 64 blocks x 32 tiles
])
def test_small_grids_split_keys_over_wavefronts(af3, oracle, B, H, L, D, live):
    """Launches with few query blocks split each block's key tiles over the wavefronts of a workgroup
    and merge the partial softmax states; every split must agree with the formula."""
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=3 * L + D)
    if isinstance(live, int):
        m[:, live:] = False
    elif live is not None:
        m[:] = False
        m[:, live[0]:live[1]] = True
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")
    dq, dk, dv, dm, _ = dev(q, k, v, m, bias)
    out = af3.dot_product_attention_cpp(dq, dk, dv, dm, torch.zeros(H, L, L, dtype=torch.bfloat16, device="cuda"))
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), np.zeros((H, L, L), np.float32))
    assert np.abs(f32np(out) - want).max() <= TOL[torch.bfloat16]


@pytest.mark.parametrize("H,L,D,bias_kind,live", [
    (16, 1536, 24, "bf16", None),          # bias through the LDS ring, one ring per pair of wavefronts
    (16, 1536, 32, "bf16", (100, 1400)),   # dead tiles at both ends
    (16, 1536, 48, "bf16", (100, 1400)),   # head_dim 48 (padded to 64) keeps one wavefront per query block
    (8, 2048, 32, "f32", None),            # fp32 bias read in place
    (16, 1000, 32, "unaligned", 900),      # bias rows that cannot take 16-byte loads: element-wise path; ragged last tile
    (16, 1536, 16, "none_live_tail", 33),  # only the first 33 keys are live
    (12, 1000, 32, "bf16", (100, 900)),    # 384 query blocks: workgroups of four computing wavefronts; ragged last tile, dead tiles at both ends
    (10, 1000, 32, "f32", None),           # the same with an fp32 bias read in place
    (10, 1000, 16, "unaligned", 900),      # ... and with bias rows that cannot take 16-byte loads
    (9, 1056, 24, "bf16", 70),             # 297 blocks, 17 key tiles of which two are live: the loading wavefronts have nothing to fetch after the first two
    (9, 1056, 24, "bf16", 150),            # three live tiles: the walk ends inside the loading wavefronts' first requests
    (9, 1056, 24, "bf16", 250),            # four live tiles: exactly what is in flight behind the first barrier
    (16, 1536, 32, "bf16", 300),           # five live tiles = the ring's length (eight computing wavefronts)
])
def test_long_rows_pair_up_wavefronts_on_shared_tiles(af3, oracle, H, L, D, bias_kind, live):
    """B = 1 with 512..1024 query blocks and at least 8 key tiles: two wavefronts share each query block and the workgroup's
    K/V tiles, each taking 32 of every 64 keys; their partial softmax states are merged at the end."""
    q, k, v, m, bias = rand_inputs(1, H, L, D, torch.bfloat16, seed=L + D)
    if isinstance(live, int):
        m[:, live:] = False
    elif live is not None:
        m[:] = False
        m[:, live[0]:live[1]] = True
    if bias_kind == "f32":                # (the drop-in casts the bias to q's dtype; the lean op hands an fp32 bias to the kernel as it is)
        from af3_kernels_amd import ops
        dq, dk, dv, dm = dev(q, k, v, m)
        out = ops._dpa_forward_impl(dq, dk, dv, ops._lift_mask(dm, L), bias.float().cuda(), ops._DTYPE_CODE[torch.bfloat16], False)
        want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
        assert np.abs(f32np(out) - want).max() <= TOL[torch.bfloat16]
        return
    if bias_kind == "unaligned":
        wide = torch.zeros(H, L, L + 3, dtype=torch.bfloat16)
        wide[:, :, :L] = bias
        dq, dk, dv, dm = dev(q, k, v, m)
        out = af3.dot_product_attention_cpp(dq, dk, dv, dm, wide.cuda()[:, :, :L])       # row stride L + 3: not a multiple of 8
        want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
        assert np.abs(f32np(out) - want).max() <= TOL[torch.bfloat16]
        return
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")


def test_long_rows_with_few_heads_pick_a_variant_that_fits_in_lds(af3, oracle):
    """B*H = 1 with L = 5000: the four-wave key split with the bias ring would need more LDS than a compute unit has
    (private K/V buffers + ring + a 20 KB mask table); the launcher must pick the next variant instead of failing."""
    q, k, v, m, bias = rand_inputs(1, 1, 5000, 32, torch.bfloat16, seed=77)
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")


def test_bf16_mfma_and_fp32_fma_kernels_agree(af3):
    q, k, v, m, bias = dev(*rand_inputs(2, 4, 200, 32, torch.bfloat16, seed=5, mask="random"))
    a = af3.dot_product_attention_cpp(q, k, v, m, bias)
    b = torch.ops.af3_kernels.dpa_forward(q, k, v, m.view(torch.uint8), bias, 1, True)   # force the fp32-FMA kernel
    torch.cuda.synchronize()
    assert (a.float() - b.float()).abs().max().item() <= 2e-2


def test_reference_flags_do_not_change_results(af3):
    q, k, v, m, bias = dev(*rand_inputs(2, 4, 300, 32, torch.bfloat16, seed=6, mask="tail"))
    a = af3.dot_product_attention_cpp(q, k, v, m, bias)
    b = af3.dot_product_attention_cpp(q, k, v, m, bias, True, 64, 128)
    assert torch.equal(a, b)


def test_native_signature_op_takes_the_inverted_typed_mask(af3):
    # what the reference wrapper hands to its extension: ~mask cast to q's dtype, [B,1,1,L]
    q, k, v, m, bias = dev(*rand_inputs(2, 4, 96, 32, torch.bfloat16, seed=7, mask="random"))
    inv = (~m)[:, None, None, :].to(q.dtype)
    a = torch.ops.af3_kernels.dot_product_attention(q, k, v, inv, bias, False, 128, 1024)
    b = af3.dot_product_attention_cpp(q, k, v, m, bias)
    assert torch.equal(a, b)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_fully_dropped_row_is_mean_of_v_and_single_key_is_exact(af3, dtype):
    B, H, L, D = 3, 2, 150, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, dtype, seed=8)
    m[1, :] = False                      # every key dropped -> uniform weights over all L keys
    m[2, :] = False
    m[2, 77] = True                      # exactly one live key -> that V row, exactly
    dq, dk, dv, dm, db = dev(q, k, v, m, bias)
    out = af3.dot_product_attention_cpp(dq, dk, dv, dm, db)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    mean = v[1].float().mean(dim=1, keepdim=True).expand(H, L, D)
    assert (out[1].float().cpu() - mean).abs().max().item() <= (1e-5 if dtype == torch.float32 else 8e-3)
    one = v[2][:, 77:78, :].expand(H, L, D).float()
    # exactly that V row for fp32; for bf16 up to one output ulp (the probabilities are rounded to bf16 for the
    # matrix product while the row sum is kept in fp32)
    assert (out[2].float().cpu() - one).abs().max().item() <= (0.0 if dtype == torch.float32 else 2 ** -7 * one.abs().max().item())


def test_values_at_dropped_keys_do_not_matter(af3):
    q, k, v, m, bias = rand_inputs(2, 4, 130, 32, torch.bfloat16, seed=9, mask="random")
    dq, dk, dv, dm, db = dev(q, k, v, m, bias)
    a = af3.dot_product_attention_cpp(dq, dk, dv, dm, db)
    k2, v2 = k.clone(), v.clone()
    for b in range(2):
        k2[b][:, ~m[b], :] = 50.0        # large finite logits at dropped keys
        v2[b][:, ~m[b], :] = -1e4
    b_ = af3.dot_product_attention_cpp(dq, k2.cuda(), v2.cuda(), dm, db)
    assert torch.equal(a, b_)


@pytest.mark.parametrize("B,H,L,D,first_live", [
    (48, 4, 256, 32, 64),     # four-wave workgroups, bias through the workspace: tile 0 is dead, tile 1 is the first
    (48, 4, 256, 32, 130),    # tiles 0 and 1 are dead
    (1, 16, 768, 24, 200),    # one row, key tiles split over two wavefronts: neither starts where it would without a mask
    (1, 16, 1536, 24, 64),    # pairs of wavefronts on shared tiles, bias ring
])
def test_rows_whose_first_key_tiles_hold_no_live_key(af3, oracle, B, H, L, D, first_live):
    """The kernel requests the tile it expects to walk first before it has read the key mask; when that tile turns out to
    hold no live key the walk starts elsewhere and the tile's buffer is loaded again.  Some batch rows keep every key, so
    both outcomes occur in one launch."""
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=L + first_live)
    m[::2, :first_live] = False
    prev = af3.set_rows_kernel("never")
    try:
        run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")
    finally:
        af3.set_rows_kernel(prev)


def test_strided_inputs_and_prepadded_bias(af3, oracle):
    B, H, L, D, M = 2, 4, 100, 32, 128
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=10, mask="random")
    big = torch.zeros(B, H, M, D + 32, dtype=torch.bfloat16)          # rows with a larger pitch
    big[:, :, :L, :D] = q
    qv = big.cuda()[:, :, :L, :D]
    kv = k.cuda().transpose(0, 1).contiguous().transpose(0, 1)         # [B,H,L,D] view with permuted strides
    padded = torch.full((H, M, M), 9.0, dtype=torch.bfloat16)          # garbage outside the L x L corner
    padded[:, :L, :L] = bias
    out = af3.dot_product_attention_cpp(qv, kv, v.cuda(), m.cuda(), padded.cuda())
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
    assert np.abs(f32np(out) - want).max() <= 2e-2


def _sweep_shapes(n, seed, widths=(8, 16, 24, 32, 40, 48, 64)):
    """Seeded shapes spread over what picks a kernel variant: the number of query blocks in the launch (few:
    keys split over wavefronts; many: one wavefront per block), lengths on both sides of the 32-, 64- and
    128-key boundaries, every padded head width, the three mask forms."""
    rng = np.random.default_rng(seed)
    shapes = []
    while len(shapes) < n:
        D = int(rng.choice(widths))
        L = int(rng.choice([rng.integers(1, 130), 64 * rng.integers(1, 20) + rng.integers(-2, 3), rng.integers(130, 1300)]))
        L = max(L, 1)
        BH = int(rng.choice([1, 2, 3, 5, 8, 16, 40, 130]))
        H = int(rng.choice([h for h in (1, 2, 4, 5, 8, 16) if BH % h == 0]))
        B = BH // H
        if B * H * L * L > 12_000_000:
            continue
        shapes.append((B, H, L, D, str(rng.choice(["none", "random", "tail"])), int(rng.choice([1, 2])), int(rng.integers(1 << 30))))
    return shapes


@pytest.mark.parametrize("B,H,L,D,mask,rank,seed", _sweep_shapes(24, 777, widths=(3, 5, 8, 12, 24, 32, 33, 64, 72, 128)))
def test_fp32_seeded_shape_sweep(af3, oracle, B, H, L, D, mask, rank, seed):
    """fp32 storage: whichever of the fp32 kernels the shape selects (matrix-core or vector-FMA)."""
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.float32, seed=seed, mask=mask, mask_rank=rank)
    run_case(af3, oracle, q, k, v, m, bias)


@pytest.mark.parametrize("B,H,L,D,mask,rank,seed", _sweep_shapes(48, 20241))
def test_bf16_seeded_shape_sweep(af3, oracle, B, H, L, D, mask, rank, seed):
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=seed, mask=mask, mask_rank=rank)
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")


def _pattern_case(rng, idx):
    """One seeded case of the sweep below: shape, storage type, memory layout of q/k/v, bias pattern, mask form and
    pattern, kernel hint.  CPU tensors (views keep their strides when moved to the GPU)."""
    dtype = torch.bfloat16 if rng.random() < 0.75 else torch.float32
    D = rng.choice([8, 16, 24, 32, 32, 48, 64, 20, 40])
    L = rng.choice([1, 2, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 257, rng.randint(1, 300)])
    B = rng.choice([1, 1, 2, 3, 4, 5, 7, 9, 13, 17])
    H = rng.choice([1, 2, 4, 8])
    while B * H * L * L > 1_500_000 and B > 1:
        B //= 2
    layout = rng.choice(["bhld", "blhd", "packed"])
    g = torch.Generator().manual_seed(5000 + idx)

    def qkv():
        if layout == "bhld":
            return torch.randn(B, H, L, D, generator=g).to(dtype)
        if layout == "blhd":                                      # [B, L, H, D] storage seen as [B, H, L, D]
            return torch.randn(B, L, H, D, generator=g).to(dtype).permute(0, 2, 1, 3)
        return torch.randn(B, L, H, 3 * D, generator=g).to(dtype).permute(0, 2, 1, 3)[..., D:2 * D]   # a slice of a packed q|k|v projection

    q, k, v = qkv(), qkv(), qkv()
    bias_kind = rng.choice(["plain", "plain", "padded", "wide", "dropped_pairs", "shifted"])
    M = L + rng.choice([1, 3, 8, 29]) if bias_kind == "padded" else L
    bias = torch.randn(H, M, M, generator=g) * (5.0 if bias_kind == "wide" else 1.5)
    if bias_kind == "dropped_pairs":                              # a mask folded into the bias, at three usual magnitudes
        bias[torch.rand(bias.shape, generator=g) < 0.15] = -rng.choice([1e4, 3e4, 1e8])
    if bias_kind == "shifted":
        bias += 5.0
    bias = bias.to(dtype)
    mask_kind = rng.choice(["all", "bernoulli", "bernoulli", "tail", "leading_dropped", "rows_without_keys", "one_key", "1d"])
    mask = torch.ones(B, L, dtype=torch.bool)
    if mask_kind == "bernoulli":
        mask = torch.rand(B, L, generator=g) < rng.choice([0.05, 0.5, 0.9])
    elif mask_kind == "tail":
        for b in range(B):
            mask[b, rng.randint(0, L):] = False
    elif mask_kind == "leading_dropped":
        mask = torch.rand(B, L, generator=g) < 0.7
        for b in range(B):
            mask[b, :rng.randint(0, L)] = False
    elif mask_kind == "rows_without_keys":
        mask = torch.rand(B, L, generator=g) < 0.8
        for b in range(B):
            if rng.random() < 0.4:
                mask[b] = False
    elif mask_kind == "one_key":
        mask = torch.zeros(B, L, dtype=torch.bool)
        for b in range(B):
            mask[b, rng.randint(0, L - 1)] = True
    elif mask_kind == "1d":
        mask = torch.rand(L, generator=g) < 0.8
    mask_form = rng.choice(["bool", "typed", "b11l"])
    rows = rng.choice(["auto", "auto", "always", "never"])
    desc = f"pattern case {idx}: {dtype} B={B} H={H} L={L} D={D} layout={layout} bias={bias_kind} mask={mask_kind}/{mask_form} rows={rows}"
    return desc, q, k, v, mask, mask_form, bias, rows


@pytest.mark.parametrize("chunk", range(5))
def test_seeded_sweep_of_layouts_masks_and_bias_patterns(af3, oracle, chunk):
    """What the shape sweeps above hold fixed: q/k/v as strided views of [B, L, H, D] and packed-projection storage, the
    mask as bool / typed / [B,1,1,L] / 1-D with leading dropped tiles, rows without keys and single live keys, biases
    that are pre-padded, wide (sigma 5), shifted, or carry a folded-in mask of -1e4 / -3e4 / -1e8 at scattered pairs;
    every kernel hint.  Each case against the fp64 formula of the oracle at the storage type's tolerance."""
    import random
    rng = random.Random(9000 + chunk)
    for i in range(30):
        idx = 100 * chunk + i
        desc, q, k, v, mask, mask_form, bias, rows = _pattern_case(rng, idx)
        print(desc, flush=True)
        dm = mask.cuda()
        if mask_form == "typed":
            dm = dm.to(q.dtype)
        elif mask_form == "b11l" and mask.dim() == 2:
            dm = dm[:, None, None, :]
        prev = af3.set_rows_kernel(rows)
        try:
            out = af3.dot_product_attention_cpp(q.cuda(), k.cuda(), v.cuda(), dm, bias.cuda())
            torch.cuda.synchronize()
        finally:
            af3.set_rows_kernel(prev)
        L = q.shape[2]
        want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), mask.numpy(), f32np(bias[:, :L, :L]))
        got = f32np(out)
        assert np.isfinite(got).all(), desc
        # Query rows all of whose live keys sit on folded-in mask values are only required to be finite: their logits are
        # -1e4 .. -1e8 plus the products, which no fp32 addition resolves to the tolerance (nor does the reference's).
        live = (mask if mask.dim() == 2 else mask[None, :]).numpy()[:, None, None, :]
        usable = (live & (f32np(bias[:, :L, :L]) > -1e3)[None]).any(-1) | ~live.any(-1)       # [B, H, L]
        err = float(np.abs(got - want)[np.broadcast_to(usable, got.shape[:3])].max()) if usable.any() else 0.0
        assert err <= TOL[q.dtype], f"{desc}: max abs err {err}"


@pytest.mark.parametrize("B,H,L,D,mask,kernel", [
    (1, 2, 700, 40, "random", "fp32_mfma"),     # head_dim 40: padded to 64 columns
    (2, 3, 37, 20, "tail", "fp32_mfma"),        # odd length, head_dim 20
    (3, 4, 384, 32, "random", "fp32_mfma"),
    (2, 2, 161, 64, "tail", "fp32_mfma"),
    (1, 1, 1, 4, "none", "fp32_mfma"),          # a single key
    (1, 1, 5, 3, "none", "fp32_fma"),           # head_dim 3: rows are not 16-byte multiples -> vector-FMA kernel
    (1, 2, 130, 128, "random", "fp32_fma"),     # head_dim beyond the matrix-core kernel
])
def test_fp32_kernels_match_formula(af3, oracle, B, H, L, D, mask, kernel):
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.float32, seed=L, mask=mask)
    err = run_case(af3, oracle, q, k, v, m, bias, expect_kernel=kernel)
    assert err <= 2e-5


def test_fp32_kernels_agree_and_cover_bf16_storage(af3, oracle):
    # the two fp32 kernels on the same problem (the lean op's last argument forces the vector-FMA kernel)
    q, k, v, m, bias = dev(*rand_inputs(2, 4, 300, 32, torch.float32, seed=31, mask="random"))
    m[1] = False                                    # a batch row without any live key: mean of V in both
    a = af3.dot_product_attention_cpp(q, k, v, m, bias)
    b = torch.ops.af3_kernels.dpa_forward(q, k, v, m.view(torch.uint8), bias, 0, True)
    torch.cuda.synchronize()
    assert (a - b).abs().max().item() <= 1e-5
    assert (a[1] - v[1].mean(dim=1, keepdim=True)).abs().max().item() <= 1e-5
    # bf16 storage whose head_dim is not a multiple of 8 takes the vector-FMA kernel
    q, k, v, m, bias = rand_inputs(2, 2, 90, 20, torch.bfloat16, seed=11, mask="random")
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="fp32_fma")


def test_fp32_mfma_strided_inputs_and_large_logits(af3, oracle):
    B, H, L, D = 2, 2, 200, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.float32, seed=41, mask="tail")
    bias = bias + torch.linspace(-50.0, 70.0, L)[None, None, :]      # the running maximum moves along the row
    big = torch.zeros(B, H, L + 8, D + 32)
    big[:, :, :L, :D] = q
    qv = big.cuda()[:, :, :L, :D]                                     # rows with a larger pitch
    kv = k.cuda().transpose(0, 1).contiguous().transpose(0, 1)        # permuted batch/head strides
    assert af3.selected_kernel(qv, kv, v.cuda(), m.cuda(), bias.cuda()) == "fp32_mfma"
    out = af3.dot_product_attention_cpp(qv, kv, v.cuda(), m.cuda(), bias.cuda())
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
    assert np.abs(f32np(out) - want).max() <= 1e-4


def test_fp32_mfma_bias_rows_with_a_large_offset(af3, oracle):
    """Query rows whose biases all carry an offset of -1000 (a soft mask value): the softmax of such a row is that of the
    row without the offset, up to the rounding of one fp32 addition per logit (half an ulp of 1000: 3e-5).  Products
    accumulated on top of the bias would be rounded at that magnitude once per matrix instruction (3e-4 measured)."""
    B, H, L, D = 3, 2, 200, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.float32, seed=43, mask="random")
    g = torch.Generator().manual_seed(44)
    bias = bias * 2
    bias[:, torch.rand(L, generator=g) < 0.3, :] -= 1000.0
    run_case(af3, oracle, q, k, v, m, bias, tol=1e-4, expect_kernel="fp32_mfma")


def test_fp32_bias_and_other_dtypes_are_cast_like_the_reference(af3, oracle):
    q, k, v, m, bias = rand_inputs(2, 4, 64, 32, torch.bfloat16, seed=12, mask="tail")
    out = af3.dot_product_attention_cpp(q.cuda(), k.float().cuda(), v.float().cuda(), m.float().cuda(), bias.float().cuda())
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
    assert out.dtype == torch.bfloat16 and np.abs(f32np(out) - want).max() <= 2e-2


@pytest.mark.parametrize("B,H,L,D", [(1, 1, 1, 8), (2, 3, 1, 32), (1, 5, 33, 8), (3, 7, 129, 40), (1, 1, 64, 64)])
def test_tiny_and_odd_shapes(af3, oracle, B, H, L, D):
    """L = 1 (softmax of one key), head_dim 8, odd head counts, lengths one past a tile edge."""
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=7 * L + D, mask="none")
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")


def test_logits_far_above_the_first_tile_move_the_reference(af3, oracle):
    """The matrix-core kernel fixes its softmax reference from the first 32 keys of a row and only
    moves it when a later logit exceeds it by a wide margin.  Rows whose large logits come late (and
    grow from tile to tile) must take that path and still match the formula."""
    B, H, L, D = 2, 2, 512, 32
    q, k, v, m, bias0 = rand_inputs(B, H, L, D, torch.bfloat16, seed=99)
    # B >= 2: bias through the fp16 log2-domain workspace, whose rounding error grows with |bias|
    # (2^-12 * |bias| * log2 e in the logit), so this case keeps |bias| moderate: +20 across the row
    # (29 in log2 units, two to three reference moves at a margin of 12), an isolated spike, and one
    # row of hugely negative but equal biases (reference of large magnitude, 16-bit subtraction).
    bias = (bias0.float() + torch.linspace(-8.0, 12.0, L)[None, None, :]).to(torch.bfloat16)
    bias[:, 5, 300] = 40.0
    bias[:, 7, :] = -3.0e4
    run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")
    # B = 1: bias read in place (exact), natural-domain reference in fp32: +100 across the row and a spike of 120
    bias = (bias0.float() + torch.linspace(-40.0, 60.0, L)[None, None, :]).to(torch.bfloat16)
    bias[:, 5, 300] = 120.0
    bias[:, 7, :] = -3.0e4
    bias[:, 9, :40] = -1.0e9          # masking expressed through the bias: the first tile of the row is dead
    run_case(af3, oracle, q[:1], k[:1], v[:1], m[:1], bias, expect_kernel="bf16_mfma")
    # the same large biases with a batch: exact when the caller asks for the in-place bias
    prev = af3.set_exact_bias(True)
    try:
        run_case(af3, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")
    finally:
        af3.set_exact_bias(prev)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32], ids=["bf16", "fp32"])
def test_minus_infinity_in_the_bias_gives_that_key_weight_zero(af3, oracle, dtype):
    """An additive -inf (a mask folded into the bias) must act like the reference's add-then-softmax: weight 0 for that
    (query, key), every other key of the row unaffected, no NaN.  Covers the in-place bias (B = 1, and B >= 2 with
    set_exact_bias) and the rewritten-bias workspace (B >= 2), at entries spread over several tiles."""
    B, H, L, D = 3, 2, 200, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, dtype, seed=77, mask="random")
    g = torch.Generator().manual_seed(78)
    hole = torch.rand(H, L, L, generator=g) < 0.2
    hole[:, :, 0] = False                       # key 0 is live in every batch row: no row loses all its keys
    hole[0, 3, 1:] = True                       # a query row left with key 0 alone
    hole[1, 5, :40] = True                      # a query row whose first tile is all -inf (key 0 included: only here)
    bias = bias.masked_fill(hole, float("-inf"))
    run_case(af3, oracle, q, k, v, m, bias)                                  # B >= 2: bias workspace
    run_case(af3, oracle, q[:1], k[:1], v[:1], m[:1], bias)                  # B = 1: bias read in place
    prev = af3.set_exact_bias(True)
    try:
        run_case(af3, oracle, q, k, v, m, bias)                              # B >= 2, in place
    finally:
        af3.set_exact_bias(prev)


def test_length_beyond_the_matrix_core_limit_uses_the_fma_kernel(af3):
    """L > 8192 is outside the matrix-core kernel's mask table; the call must still work (fp32-FMA
    kernel) -- checked through rows summing to one and against a torch reference on a slice."""
    B, H, L, D = 1, 1, 8200, 32
    g = torch.Generator().manual_seed(1)
    q, k, v = [torch.randn(B, H, L, D, generator=g).to(torch.bfloat16).cuda() for _ in range(3)]
    bias = torch.zeros(H, L, L, dtype=torch.bfloat16, device="cuda")
    m = torch.ones(B, L, dtype=torch.bool, device="cuda")
    m[:, 8000:] = False
    assert af3.selected_kernel(q, k, v, m, bias) == "fp32_fma"
    out = af3.dot_product_attention_cpp(q, k, v, m, bias)
    s = (q[0, 0, :64].float() * D ** -0.5) @ k[0, 0].float().T
    s[:, 8000:] = -1e9
    want = torch.softmax(s, -1) @ v[0, 0].float()
    assert (out[0, 0, :64].float() - want).abs().max().item() <= 2e-2


# ---- the benchmark configurations at their real sizes ---------------------------------------

@pytest.mark.parametrize("name,sample_rows", [("cfg2", [0, 191, 383]), ("cfg3", [0]), ("cfg4", [0, 400, 767]), ("fp32_n768", [0, 63])])
def test_named_configs_full_size(af3, oracle, name, sample_rows):
    """Runs the whole configuration on the GPU; the oracle checks sampled batch rows (every batch
    row is an independent problem sharing the bias), properties check the rest."""
    from af3_kernels_amd.synthetic import CASES, make_inputs
    case = CASES[name]
    q, k, v, mask, bias = make_inputs(case)
    dq, dk, dv, dm, db = dev(q, k, v, mask, bias)
    assert af3.selected_kernel(dq, dk, dv, dm, db) == ("fp32_mfma" if case.io_dtype == "fp32" else "bf16_mfma")
    print(f"{name}: full size {tuple(q.shape)}", flush=True)
    out = af3.dot_product_attention_cpp(dq, dk, dv, dm, db)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    for b in sample_rows:
        mrow = mask if mask.dim() == 1 else mask[b:b + 1]
        want = oracle.dpa_formula(f32np(q[b:b + 1]), f32np(k[b:b + 1]), f32np(v[b:b + 1]), mrow.numpy(), f32np(bias))
        err = np.abs(f32np(out[b:b + 1]) - want).max()
        assert err <= case.tol, (name, b, err)
    # rows of the softmax sum to one: v = 1 gives 1 everywhere (checks every row of the full problem)
    ones = af3.dot_product_attention_cpp(dq, dk, torch.ones_like(dv), dm, db)
    assert (ones.float() - 1).abs().max().item() <= (1e-5 if case.io_dtype == "fp32" else 8e-3)
    # a per-(head, query) shift of the bias leaves the result unchanged; the bias is first snapped to multiples of
    # 1/8 so that bias + shift is exact in bf16 and the two runs see exactly shifted logits
    coarse = (db.float() * 8).round() / 8
    shift = torch.randint(-2, 3, (case.H, case.L, 1), device="cuda").float() * 4
    base = af3.dot_product_attention_cpp(dq, dk, dv, dm, coarse.to(db.dtype))
    shifted = af3.dot_product_attention_cpp(dq, dk, dv, dm, (coarse + shift).to(db.dtype))
    assert (shifted.float() - base.float()).abs().max().item() <= (1e-4 if case.io_dtype == "fp32" else 2e-2)   # bf16: one ulp of an output near 2
    # output is a convex combination of V rows
    vmax = dv.float().amax(dim=2, keepdim=True)
    vmin = dv.float().amin(dim=2, keepdim=True)
    assert (out.float() <= vmax + 1e-2).all() and (out.float() >= vmin - 1e-2).all()


# ---- the kernel for batches that share a bias (four batch rows per wavefront) -----------------------------------------
# Large launches take it by themselves (the named configs above do); here it is forced on small and awkward shapes.

@pytest.mark.parametrize("B,H,L,D,rows", [(1, 2, 192, 24, "never"), (3, 2, 64, 32, "never"), (5, 2, 192, 32, "always"), (17, 1, 64, 32, "always")])
def test_key_mask_rows_that_are_not_4_byte_aligned(af3, oracle, B, H, L, D, rows):
    """The kernels read 4-byte aligned mask rows four keys per load and anything else byte by byte: a mask that is a view
    into a wider tensor (odd storage offset, odd row stride) must give what its contiguous copy gives."""
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=L + B, mask="random")
    wide = torch.zeros(B, L + 7, dtype=torch.bool)
    wide[:, 3:3 + L] = m
    dq, dk, dv, db, dwide = dev(q, k, v, bias, wide)
    view = dwide[:, 3:3 + L]
    assert view.data_ptr() % 4 != 0 and view.stride(0) % 4 != 0
    prev = af3.set_rows_kernel(rows)
    try:
        got_view = af3.dot_product_attention_cpp(dq, dk, dv, view, db)
        got_copy = af3.dot_product_attention_cpp(dq, dk, dv, view.contiguous(), db)
    finally:
        af3.set_rows_kernel(prev)
    torch.cuda.synchronize()
    assert torch.equal(got_view, got_copy)
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
    assert float(np.abs(f32np(got_view) - want).max()) <= TOL[torch.bfloat16]


@pytest.fixture
def rows_kernel(af3):
    prev = af3.set_rows_kernel("always")
    yield af3
    af3.set_rows_kernel(prev)


@pytest.mark.parametrize("B,H,L,D,mask,rank", [
    (4, 4, 128, 32, "none", 2), (5, 2, 200, 32, "random", 2), (8, 4, 384, 32, "tail", 2), (7, 3, 37, 24, "random", 2),
    (4, 1, 65, 16, "tail", 1), (9, 4, 1000, 32, "random", 2), (4, 2, 96, 8, "none", 1), (6, 16, 256, 24, "tail", 1),
    (13, 1, 1, 32, "none", 2), (4, 5, 33, 32, "random", 2), (12, 4, 1491, 32, "random", 2),
    (2, 4, 128, 32, "none", 2), (3, 2, 200, 32, "random", 2), (5, 16, 256, 24, "tail", 1), (6, 3, 36, 24, "random", 2),   # groups of two and three rows
    (17, 2, 100, 32, "random", 2), (18, 2, 37, 32, "random", 2), (19, 1, 64, 16, "tail", 2),                          # 4 ... 4 + 3 + 2, + 2, + 3
    (16, 1, 1024, 32, "random", 2), (18, 2, 992, 24, "tail", 2), (5, 16, 1536, 24, "random", 2),   # few workgroups, long rows
])
def test_shared_bias_kernel_matches_formula(rows_kernel, oracle, B, H, L, D, mask, rank):
    """Every way the batch is cut into groups of four, three and two rows, with the bias through the rewritten workspace
    (16 batch rows and more) or read in place (fewer; lengths that are not multiples of 4 then leave the call to the
    one-row kernel), and again without a workspace at all (set_exact_bias: in place whenever the layout allows)."""
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=5 * L + D + B, mask=mask, mask_rank=rank)
    if B >= 6:
        m = m.clone() if m.dim() == 2 else m
        if m.dim() == 2:
            m[B - 1, :] = False                # a batch row without live keys in the last (partial) group
    run_case(rows_kernel, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")
    prev = rows_kernel.set_exact_bias(True)
    try:
        run_case(rows_kernel, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")
    finally:
        rows_kernel.set_exact_bias(prev)


@pytest.mark.parametrize("pattern", ["even_tiles", "odd_tiles", "first_40", "last_tile", "row_without_keys"])
def test_shared_bias_kernel_with_lopsided_masks(rows_kernel, oracle, pattern):
    """Masks that leave whole key tiles without a live key (every other tile, everything but the first 40 keys, everything
    but the last tile) or a batch row without any: the walk stops behind the last live key of the group, dead tiles in
    between contribute exactly nothing, and both bf16 kernels agree."""
    B, H, L, D = 3, 2, 800, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=len(pattern))
    tile = torch.arange(L) // 32
    if pattern == "even_tiles":
        m[:] = (tile % 2 == 0)[None, :]
    elif pattern == "odd_tiles":
        m[:] = (tile % 2 == 1)[None, :]
        m[1] = (tile % 2 == 0)
    elif pattern == "first_40":
        m[:, 40:] = False
    elif pattern == "last_tile":
        m[:] = False
        m[:, 790:] = True
    else:
        m[1, :] = False
    run_case(rows_kernel, oracle, q, k, v, m, bias, expect_kernel="bf16_mfma")
    dq, dk, dv, dm, db = dev(q, k, v, m, bias)
    a = rows_kernel.dot_product_attention_cpp(dq, dk, dv, dm, db)
    rows_kernel.set_rows_kernel("never")
    b = rows_kernel.dot_product_attention_cpp(dq, dk, dv, dm, db)
    rows_kernel.set_rows_kernel("always")
    assert (a.float() - b.float()).abs().max().item() <= 2e-2


def test_shared_bias_kernel_applies_the_output_gate(rows_kernel, oracle):
    from af3_kernels_amd import ops, _lib
    B, H, L, D = 6, 4, 200, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=7, mask="random")
    g = torch.randn(B, H, L, D, generator=torch.Generator().manual_seed(8)).to(torch.bfloat16)
    out = ops._dpa_forward_impl(q.cuda(), k.cuda(), v.cuda(), ops._lift_mask(m.cuda(), L), bias.cuda(), _lib.AF3_BF16, False, gate=g.cuda())
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias)) / (1.0 + np.exp(-f32np(g)))
    assert np.abs(f32np(out) - want).max() <= 2e-2


def test_shared_bias_kernel_agrees_with_the_one_row_kernel(af3):
    """Same arithmetic in both kernels (bf16 products, fp32 accumulation, bf16 probabilities); they differ in the rounding of
    the bias (fp32 here, fp16 in the one-row kernel's workspace) and in summation order."""
    q, k, v, m, bias = dev(*rand_inputs(8, 4, 300, 32, torch.bfloat16, seed=31, mask="random"))
    af3.set_rows_kernel("always")
    a = af3.dot_product_attention_cpp(q, k, v, m, bias).float()
    af3.set_rows_kernel("never")
    b = af3.dot_product_attention_cpp(q, k, v, m, bias).float()
    af3.set_rows_kernel("auto")
    assert (a - b).abs().max().item() <= 1.6e-2 and (a - b).abs().mean().item() <= 1e-3


def test_shared_bias_kernel_edge_cases(rows_kernel, oracle):
    af3 = rows_kernel
    B, H, L, D = 9, 2, 150, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=41, mask="random")
    m[1, :] = False                       # a batch row without live keys: mean of V, whatever the bias says
    m[2, :] = False
    m[2, 77] = True                       # a single live key: that V row
    m[5, :64] = False                     # the first tiles of a row are dead: its reference starts at the mask constant
    m[6, 100:] = False                    # keys behind the last live key of every row of a group are not walked
    m[7, 100:] = False
    m[4, 100:] = False
    out = af3.dot_product_attention_cpp(*dev(q, k, v, m, bias)).float().cpu()
    assert torch.isfinite(out).all()
    want = torch.from_numpy(oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias)))
    assert (out - want).abs().max().item() <= 2e-2
    mean = v[1].float().mean(dim=1, keepdim=True).expand(H, L, D)
    assert (out[1] - mean).abs().max().item() <= 1.6e-2
    one = v[2][:, 77:78, :].expand(H, L, D).float()
    assert (out[2] - one).abs().max().item() <= 2 ** -7 * one.abs().max().item()
    # values at dropped keys do not matter, NaN and infinity included in K and V... as long as they are finite in K (0 * inf)
    k2, v2 = k.clone(), v.clone()
    for b in range(B):
        k2[b][:, ~m[b], :] = 50.0
        v2[b][:, ~m[b], :] = -1e4
    again = af3.dot_product_attention_cpp(*dev(q, k2, v2, m, bias)).float().cpu()
    live_rows = [b for b in range(B) if m[b].any()]
    assert torch.equal(again[live_rows], out[live_rows])
    # fp32 bias (exact in this kernel's workspace), fp32 output through the lean op, no bias at all, strided inputs
    run_case(af3, oracle, q, k, v, m, bias.float())
    dq, dk, dv, dm = dev(q, k, v, m)
    nob = af3.dot_product_attention_cpp(dq, dk, dv, dm, None)
    want0 = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), np.zeros((H, L, L), np.float32))
    assert np.abs(f32np(nob) - want0).max() <= 2e-2
    big = torch.randn(B, H, L, 3 * D, generator=torch.Generator().manual_seed(42)).to(torch.bfloat16)
    qs, ks, vs = big[..., :D], big[..., D:2 * D], big[..., 2 * D:]
    run_case(af3, oracle, qs, ks, vs, m, bias)


def test_shared_bias_kernel_moves_its_reference(rows_kernel, oracle):
    """Logits that grow along the row, isolated spikes, rows of hugely negative biases, masking expressed through the bias,
    the reference harness's large-mean recipe and -inf entries: the rare path of every one of the four row chains."""
    af3 = rows_kernel
    B, H, L, D = 6, 2, 512, 32
    q, k, v, m, bias0 = rand_inputs(B, H, L, D, torch.bfloat16, seed=99)
    bias = (bias0.float() + torch.linspace(-40.0, 60.0, L)[None, None, :]).to(torch.bfloat16)
    bias[:, 5, 300] = 120.0
    bias[:, 7, :] = -3.0e4
    bias[:, 9, :40] = -1.0e9
    bias[:, 11, 1:] = float("-inf")
    run_case(af3, oracle, q, k, v, m, bias)
    g = torch.Generator().manual_seed(1896)
    q, k, v = [(torch.randn(B, H, L, D, generator=g) * 2 + 3).to(torch.bfloat16) for _ in range(3)]
    bias = (torch.randn(H, L, L, generator=g) * 2 + 3).to(torch.bfloat16)
    # outputs are 3 +- 2 here and logits 50 +- 20, so the softmax is nearly one-hot and the bf16 rounding of the scaled q alone
    # moves single weights by percents: judged by the harness's own relative-L1 measure (examples/dot_product_attention.py:129-134)
    out = f32np(af3.dot_product_attention_cpp(*dev(q, k, v, m, bias)))
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
    assert np.isfinite(out).all()
    assert np.abs(out - want).sum() / np.abs(want).sum() <= 5e-3
    assert np.abs(out - want).max() <= 0.25


@pytest.mark.parametrize("B,L,bias_dtype", [(6, 320, torch.bfloat16), (6, 324, torch.bfloat16), (20, 324, torch.bfloat16), (20, 320, torch.float32)],
                         ids=["bias_staged_through_lds", "bias_read_in_place", "bias_workspace", "bias_workspace_from_fp32"])
def test_shared_bias_kernel_leading_dead_tiles_and_hugely_negative_bias_rows(rows_kernel, oracle, B, L, bias_dtype):
    """A batch row whose leading key tiles hold no live key fixes its softmax reference at its first tile that does.  Query
    rows whose biases are -3e4, -1e9 or -inf throughout (padded queries masked through the bias) then still get a finite
    result -- the softmax over their live keys, uniform where nothing distinguishes them -- exactly as for batch rows whose
    first tile is live, and as the one-row kernel gives."""
    af3 = rows_kernel
    H, D = 2, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=1234 + B, mask="random")
    m[1, :64] = False        # two leading tiles without a live key
    m[3, :32] = False        # one
    m[2, :300] = False       # nearly everything: the reference is fixed in the row's last tile but one
    m[:, 310] = True
    bias = bias.to(bias_dtype)
    bias[:, 5, :] = -3.0e4
    bias[:, 6, :] = -1.0e9
    bias[:, 7, :] = float("-inf")
    bias[:, 40, :] = -3.0e4
    bias[:, 40, 200] = -2.9e4     # one key stands out by far
    try:
        out = af3.dot_product_attention_cpp(*dev(q, k, v, m, bias)).float().cpu()
        af3.set_rows_kernel("never")
        other = af3.dot_product_attention_cpp(*dev(q, k, v, m, bias)).float().cpu()
    finally:
        af3.set_rows_kernel("always")
    assert torch.isfinite(out).all() and torch.isfinite(other).all()
    # The kernels clamp -1e9 and -inf in the bias to a large finite value, so such a query row is the softmax of q.k over its
    # live keys, and dropped keys keep weight exactly 0.  The formula says the same once these rows hold a value that stays
    # apart from its masked_fill(-1e9) (at -1e9 itself a dropped key would tie with the live ones; a row of -inf is NaN).
    fbias = bias.float().clone()
    fbias[:, 6, :] = -1.0e8
    fbias[:, 7, :] = -1.0e8
    want = torch.from_numpy(oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), fbias.numpy()))
    assert (out - want).abs().max().item() <= 2e-2
    assert (out - other).abs().max().item() <= 2e-2
    # the query row with one outstanding key returns that key's V row (where the key is live)
    for b in range(B):
        if m[b, 200]:
            assert (out[b, :, 40, :] - v[b, :, 200, :].float()).abs().max().item() <= 2 ** -7 * v[b, :, 200, :].float().abs().max().item() + 1e-6


# ---- element-wise kernels -------------------------------------------------------------------

def test_convert_matches_torch_casts(af3):
    g = torch.Generator().manual_seed(3)
    x = torch.cat([torch.randn(100003, generator=g) * 7, torch.tensor([0.0, -0.0, 1.00390625, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8, 3.3895e38, 1e-40, float("inf")])])
    got = af3.convert(x.cuda(), torch.bfloat16)
    assert torch.equal(got.cpu().view(torch.int16), x.to(torch.bfloat16).view(torch.int16))
    back = af3.convert(got, torch.float32)
    assert torch.equal(back.cpu(), x.to(torch.bfloat16).float())
    codes = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn)
    want = codes.float()
    got = af3.convert(codes.cuda(), torch.float32).cpu()
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan) and torch.equal(got[~nan], want[~nan])
    assert torch.equal(af3.convert(codes.cuda(), torch.bfloat16).cpu()[~nan], want.to(torch.bfloat16)[~nan])


def test_convert_e5m2_matches_torch_casts_bit_for_bit(af3):
    """The e5m2 pair of the cast functors (src/csrc/xsmm_functors.h:211-217): every code decodes like torch.float8_e5m2, and
    fp32 / bf16 values -- any bit pattern, ties between representable values and their neighbours, subnormals, the overflow
    threshold, infinities -- encode to exactly torch's bits (one rounding to nearest even, overflow to infinity)."""
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e5m2).float()
    nan = torch.isnan(want)
    got = af3.convert(codes.view(torch.float8_e5m2).cuda(), torch.float32).cpu()
    assert torch.equal(torch.isnan(got), nan) and torch.equal(got[~nan], want[~nan])
    got16 = af3.convert(codes.view(torch.float8_e5m2).cuda(), torch.bfloat16).cpu()
    assert torch.equal(got16[~nan].float(), want[~nan])
    g = torch.Generator().manual_seed(5)
    bits = torch.randint(-2 ** 31, 2 ** 31 - 1, (300001,), generator=g, dtype=torch.int64).to(torch.int32).view(torch.float32)
    finite = want[torch.isfinite(want)].sort().values
    mid = (finite[:-1] + finite[1:]) / 2
    x = torch.cat([bits, torch.randn(100003, generator=g) * 3, mid, torch.nextafter(mid, torch.tensor(float("inf"))), torch.nextafter(mid, torch.tensor(float("-inf"))),
                   torch.tensor([0.0, -0.0, 2.0 ** -17, 2.0 ** -16, 1.5 * 2.0 ** -16, 57344.0, 61439.99, 61440.0, 65535.0, 65536.0, float("inf"), float("-inf")])])
    x = x[~torch.isnan(x)]
    for src in (x, x.to(torch.bfloat16)):
        got = af3.convert(src.cuda(), torch.float8_e5m2).cpu().view(torch.uint8)
        assert torch.equal(got, src.to(torch.float8_e5m2).view(torch.uint8))
    assert (af3.convert(torch.tensor([float("nan")]).cuda(), torch.float8_e5m2).cpu().view(torch.uint8) & 0x7f).item() > 0x7c


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_quantize_fp8_per_tensor_scale(af3, dtype):
    g = torch.Generator().manual_seed(4)
    x = (torch.randn(3, 2, 40, 24, generator=g) * 3).to(dtype)
    q8, descale = af3.quantize_fp8_e4m3(x.cuda(), pre_scale=0.5)
    amax = x.float().abs().max().item() * 0.5
    scale = 2.0 ** np.floor(np.log2(448.0 / amax))
    assert descale.item() == pytest.approx(1.0 / scale, rel=0, abs=0)
    want = (x.float() * 0.5 * scale).clamp(-448, 448).to(torch.float8_e4m3fn)
    assert torch.equal(q8.cpu().view(torch.uint8), want.view(torch.uint8))
    # transposed form: last two axes swapped
    t8, d2 = af3.quantize_fp8_e4m3(x.cuda(), transpose_last2=True)
    scale1 = 2.0 ** np.floor(np.log2(448.0 / (amax * 2)))
    want_t = (x.float() * scale1).clamp(-448, 448).to(torch.float8_e4m3fn).transpose(-1, -2)
    assert t8.shape == (3, 2, 24, 40) and torch.equal(t8.cpu().view(torch.uint8), want_t.contiguous().view(torch.uint8))
    assert d2.item() == 1.0 / scale1


@pytest.mark.parametrize("shape", [(2, 2, 37, 24), (1, 3, 5, 8), (2, 1, 130, 48), (1, 2, 64, 20)], ids=str)
def test_quantize_fp8_transposed_ragged_rows(af3, shape):
    """Transposed e4m3 of bf16 rows whose count is no multiple of four (the last row quad of a matrix is partly padding),
    with head sizes of whole 16-byte chunks (the 4-rows-by-8-columns path) and one that is not."""
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 2).to(torch.bfloat16)
    t8, d = af3.quantize_fp8_e4m3(x.cuda(), transpose_last2=True)
    scale = 2.0 ** np.floor(np.log2(448.0 / x.float().abs().max().item()))
    want = (x.float() * scale).clamp(-448, 448).to(torch.float8_e4m3fn).transpose(-1, -2).contiguous()
    assert t8.shape == want.shape and d.item() == 1.0 / scale
    assert torch.equal(t8.cpu().contiguous().view(torch.uint8), want.view(torch.uint8))


def test_pad_and_vnni_repack(af3, oracle):
    x = torch.arange(2 * 3 * 5, dtype=torch.float32).reshape(2, 3, 5).cuda()
    y = af3.pad_and_align_tensor(x, (2, 4, 8), True, 1.0)
    want = torch.ones(2, 4, 8)
    want[:, :3, :5] = x.cpu()
    assert torch.equal(y.cpu(), want)
    assert af3.pad_and_align_tensor(x, (2, 3, 5)) is x                # already padded, contiguous, aligned: returned as is
    b = torch.randn(4, 37, 37).to(torch.bfloat16).cuda()
    pb = af3.pad_and_align_tensor(b, (4, 128, 128))
    assert torch.equal(pb[:, :37, :37], b) and pb[:, 37:, :].abs().sum() == 0 and pb[:, :, 37:].abs().sum() == 0
    w = torch.randn(16, 24).to(torch.bfloat16)
    got = af3.vnni_repack_tensor(w.cuda(), 2, 8).cpu().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, oracle.vnni_repack(w.view(torch.int16).numpy().view(np.uint16), 8))
    with pytest.raises(ValueError):
        af3.vnni_repack_tensor(w.cuda(), 2, 7)


def test_timers_report_calls(af3, capsys):
    q, k, v, m, bias = dev(*rand_inputs(1, 2, 64, 32, torch.bfloat16, seed=1))
    af3.reset_debug_timers()
    for _ in range(3):
        af3.dot_product_attention_cpp(q, k, v, m, bias)
    af3.print_debug_timers()
    assert "calls=3" in capsys.readouterr().out


# ---- fp8 (e4m3) matrix-core path ------------------------------------------------------------
# No reference behaviour exists for fp8 (the reference's e4m3 converters are unimplemented asserts); the only pin is
# the fp32 formula on the un-quantised inputs within 6e-2.

@pytest.mark.parametrize("B,H,L,D,mask,rank", [
    (2, 4, 128, 32, "none", 2),
    (2, 16, 256, 24, "tail", 1),      # diffusion shape: head_dim 24, 1-D mask
    (3, 4, 200, 32, "random", 2),
    (1, 2, 37, 24, "random", 1),      # ragged length: transposed V rows padded to 16 bytes
    (2, 2, 130, 48, "tail", 2),
    (1, 16, 1536, 24, "tail", 1),     # one sample of the diffusion-transformer case
])
def test_fp8_mfma_matches_formula(af3, oracle, B, H, L, D, mask, rank):
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=3 * L + D, mask=mask, mask_rank=rank)
    dq, dk, dv, dm, db = dev(q, k, v, m, bias)
    print(f"fp8 case {(B, H, L, D)}", flush=True)
    plain = af3.dot_product_attention_fp8(dq, dk, dv, dm, db, compensated=False)
    comp = af3.dot_product_attention_fp8(dq, dk, dv, dm, db)
    torch.cuda.synchronize()
    assert comp.dtype == torch.bfloat16 and comp.shape == q.shape
    plain, comp = f32np(plain), f32np(comp)
    assert np.isfinite(plain).all() and np.isfinite(comp).all()
    vq = oracle.fake_quantize_e4m3_pow2(f32np(v))
    # (1) kernel logic, single-term product: against the formula on the inputs as the kernel sees them (q, k, v through
    # the same per-tensor e4m3 quantiser; q carries D^-1/2).  What remains is the e4m3 rounding of P and the bf16 output.
    qq = oracle.fake_quantize_e4m3_pow2(f32np(q), D ** -0.5) * D ** 0.5
    kq = oracle.fake_quantize_e4m3_pow2(f32np(k))
    want_q = oracle.dpa_formula(qq, kq, vq, m.numpy(), f32np(bias))
    assert np.abs(plain - want_q).max() <= 4e-2, np.abs(plain - want_q).max()
    assert np.abs(plain - want_q).mean() <= 6e-3
    # (2) compensated product (the default): q and k are effectively exact, only v and P are e4m3
    want_v = oracle.dpa_formula(f32np(q), f32np(k), vq, m.numpy(), f32np(bias))
    assert np.abs(comp - want_v).max() <= 4e-2, np.abs(comp - want_v).max()
    # (3) the stated fp8 budget against the formula on the un-quantised inputs: 6e-2 at diffusion-sized L.  Short
    # rows, where a single key can carry most of the weight, see the e4m3 rounding of that V row and of its
    # probability directly (2^-4 relative each): with q and k exact, those two roundings alone move these very
    # inputs by 0.07 - 0.10 (tests/test_oracle_pins.py::test_fp8_short_row_error_budget_is_the_e4m3_rounding_of_p_and_v
    # computes it on the CPU for the same seeds), so no e4m3 kernel meets 6e-2 there; the bound is that test's 0.15.
    want = oracle.dpa_formula(f32np(q), f32np(k), f32np(v), m.numpy(), f32np(bias))
    err = np.abs(comp - want).max()
    assert err <= (6e-2 if L >= 1024 else 0.15), err
    assert np.abs(comp - want).mean() <= (6e-3 if L >= 128 else 1.2e-2)
    assert np.abs(comp - want).mean() < np.abs(plain - want).mean()    # the residual terms help


def test_fp8_fully_dropped_row_and_single_key(af3):
    B, H, L, D = 3, 2, 150, 32
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=21)
    m[1, :] = False
    m[2, :] = False
    m[2, 77] = True
    out = af3.dot_product_attention_fp8(*dev(q, k, v, m, bias)).float().cpu()
    assert torch.isfinite(out).all()
    mean = v[1].float().mean(dim=1, keepdim=True).expand(H, L, D)
    assert (out[1] - mean).abs().max().item() <= 3e-2          # V itself is quantised to e4m3 (3 mantissa bits)
    one = v[2][:, 77:78, :].expand(H, L, D).float()
    assert (out[2] - one).abs().max().item() <= 2 ** -4 * one.abs().max().item()


def test_cfg5_fp8_full_size(af3, oracle):
    from af3_kernels_amd.synthetic import CASES, make_inputs
    case = CASES["cfg5"]
    q, k, v, mask, bias = make_inputs(case)
    out = af3.dot_product_attention_fp8(*dev(q, k, v, mask, bias))
    torch.cuda.synchronize()
    assert torch.isfinite(out).all()
    for b in (0, 4):
        want = oracle.dpa_formula(f32np(q[b:b + 1]), f32np(k[b:b + 1]), f32np(v[b:b + 1]), mask.numpy(), f32np(bias))
        err = np.abs(f32np(out[b:b + 1]) - want).max()
        assert err <= case.tol, (b, err)


# ---- HIP graph capture ------------------------------------------------------------------------

def test_calls_can_be_captured_in_a_hip_graph_and_replayed(af3):
    """The entry points only enqueue kernels on the given stream (no allocation, no synchronisation,
    no memset nodes), so a call can be recorded into a HIP graph.  Every replay, with eager work and
    synchronisations in between and fresh inputs copied into the captured buffers, must reproduce
    the eager result bit for bit."""
    B, H, L, D = 3, 4, 200, 32
    q, k, v, m, bias = dev(*rand_inputs(B, H, L, D, torch.bfloat16, seed=21, mask="random"))
    sq, sk, sv = q.clone(), k.clone(), v.clone()
    af3.dot_product_attention_cpp(sq, sk, sv, m, bias)          # warm-up outside the capture (library load)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            out = af3.dot_product_attention_cpp(sq, sk, sv, m, bias)
    torch.cuda.synchronize()
    for rep in range(4):
        g = torch.Generator().manual_seed(100 + rep)
        nq, nk, nv = [torch.randn(B, H, L, D, generator=g).to(torch.bfloat16).cuda() for _ in range(3)]
        sq.copy_(nq), sk.copy_(nk), sv.copy_(nv)
        graph.replay()
        torch.cuda.synchronize()
        eager = af3.dot_product_attention_cpp(nq, nk, nv, m, bias)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager call"


def test_fp8_k_rows_are_not_read_past_their_allocation(af3, oracle):
    """head_dim 24: K rows are fetched in 16-byte chunks, so the last chunk of the last row would reach
    8 bytes past the tensor.  The kernel's buffer ends at the last valid byte and must return zeros
    beyond it: k and its residual are placed directly in front of e4m3 NaN bytes (0x7F), which would
    poison the result if they were read."""
    import ctypes
    from af3_kernels_amd import ops
    B, H, L, D = 2, 3, 200, 24
    q, k, v, m, bias = rand_inputs(B, H, L, D, torch.bfloat16, seed=77, mask="random")
    dq, dk, dv, dm, db = dev(q, k, v, m, bias)
    want = af3.dot_product_attention_fp8(dq, dk, dv, dm, db)
    scratch = torch.zeros(6, dtype=torch.float32, device="cuda")
    q8, _, q_lo = af3.quantize_fp8_e4m3(dq, pre_scale=D ** -0.5, descale_out=scratch[3:4], with_residual=True, amax_buf=scratch[0:1])
    k8, _, k_lo = af3.quantize_fp8_e4m3(dk, descale_out=scratch[4:5], with_residual=True, amax_buf=scratch[1:2])
    v8t, _ = af3.quantize_fp8_e4m3(dv, transpose_last2=True, descale_out=scratch[5:6], amax_buf=scratch[2:3])

    def poisoned(t):
        arena = torch.full((t.numel() + 64,), 0x7F, dtype=torch.uint8, device="cuda")
        arena[:t.numel()] = t.contiguous().view(torch.uint8).reshape(-1)
        return arena, arena[:t.numel()].view(torch.float8_e4m3fn).view(t.shape)

    a1, k8p = poisoned(k8)
    a2, klop = poisoned(k_lo)
    out = torch.empty_like(dq)
    keep = ops._lift_mask(dm, L)
    p = ops._fill_params(q8, k8p, v8t, keep, db, out, ops.AF3_FP8_E4M3, False, descales=scratch[3:6], softmax_scale=1.0)
    p.q_lo, p.k_lo = q_lo.data_ptr(), klop.data_ptr()
    print("fp8 forward on k tensors followed by NaN bytes", flush=True)
    rc = af3._lib.load().af3_dpa_forward(ctypes.byref(p), torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 0
    assert torch.isfinite(out).all()
    assert torch.equal(out, want)
