"""The reference harness's own cases on the GPU, through the package name the harness imports.

examples/dot_product_attention.py draws its inputs with seed 1896 as randn * 2 + 3 in bfloat16 (:17, :95-109), uses an
all-ones mask and six shape presets (:47-85), and prints the relative L1 distance between the formula and the compiled op
(:129-134) without a threshold.  Logits of that recipe have a large mean (about 50 +- 20 in natural units), far above what
the bf16 kernel's first-tile softmax reference expects, so every row takes the kernel's reference-moving path.  Each preset
is run at full size; sampled batch rows are compared with the float64 formula using the harness's metric, and the bound is
twice what the CPU restatement of the reference's own bf16 arithmetic scores on the same rows.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

SEED, SCALE, BIAS = 1896, 2.0, 3.0      # examples/dot_product_attention.py:17, :97-98
PRESETS = {                               # examples/dot_product_attention.py:49-85
    1: ((37, 4, 37, 32), (37, 37)),
    2: ((2048, 4, 2048, 32), (2048, 2048)),
    3: ((1491, 4, 1491, 32), (1491, 1491)),
    4: ((1, 16, 37, 48), (37,)),
    5: ((1, 16, 128, 48), (128,)),
    6: ((1, 16, 1491, 24), (1491,)),
}


def _f32(t):
    return t.detach().float().cpu().numpy()


@pytest.mark.parametrize("set_size", sorted(PRESETS))
def test_reference_harness_preset(oracle, set_size):
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import af3_kernels                                   # the alias package: the harness's own import line
    from af3_kernels import dot_product_attention_cpp
    qkv_shape, mask_shape = PRESETS[set_size]
    B, H, L, D = qkv_shape
    torch.manual_seed(SEED)
    q = torch.randn(qkv_shape, dtype=torch.bfloat16) * SCALE + BIAS
    k = torch.randn(qkv_shape, dtype=torch.bfloat16) * SCALE + BIAS
    v = torch.randn(qkv_shape, dtype=torch.bfloat16) * SCALE + BIAS
    bias = torch.randn((H, L, L), dtype=torch.bfloat16) * SCALE + BIAS
    mask = torch.ones(mask_shape, dtype=torch.bool)
    print(f"harness preset {set_size}: qkv {qkv_shape}", flush=True)
    af3_kernels.reset_debug_timers()
    out = dot_product_attention_cpp(q.cuda(), k.cuda(), v.cuda(), mask.cuda(), bias.cuda(), False, 128, 1024)   # USE_FLASH, BLK_SZ, FLASH_SZ as in :89-92
    torch.cuda.synchronize()
    assert out.shape == q.shape and out.dtype == torch.bfloat16
    assert torch.isfinite(out).all()
    rows = sorted({0, B // 2, B - 1})
    num = den = ref_num = 0.0
    for b in rows:
        sl = slice(b, b + 1)
        m = mask.numpy() if mask.dim() == 1 else mask[sl].numpy()
        want = oracle.dpa_formula(_f32(q[sl]), _f32(k[sl]), _f32(v[sl]), m, _f32(bias))
        ref = oracle.dpa_reference(_f32(q[sl]), _f32(k[sl]), _f32(v[sl]), m, _f32(bias), dtype=oracle.BF16, BLK_SZ=128)
        got = _f32(out[sl])
        num += np.abs(got - want).sum()
        ref_num += np.abs(ref - want).sum()
        den += np.abs(want).sum()
        # rows of V are 3 +- 2: the result is a convex combination of them
        assert got.max() <= _f32(v[sl]).max() + 0.05 and got.min() >= _f32(v[sl]).min() - 0.05
    diff, ref_diff = num / den, ref_num / den               # the harness's "Diff" (as a fraction)
    print(f"  Diff {100 * diff:.5f} %   (reference arithmetic restated on the CPU: {100 * ref_diff:.5f} %)", flush=True)
    assert diff <= 2.0 * ref_diff + 1e-6, (diff, ref_diff)
    assert diff <= 5e-3                                      # measured 0.17 - 0.21 %; the reference's bf16 logits alone cost 1.3 - 2.4 % here
