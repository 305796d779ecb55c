"""Writes the golden vectors under tests/golden/ (run from the repo root:
`python tests/golden/make_golden.py`).

The reference holds no fixtures for this path and cannot be imported (its extension needs
libxsmm), so the expected outputs are computed here by the float64 closed form of the harness
formula (examples/dot_product_attention.py:20-43, restated in oracle/dpa_numpy.py) on seeded
inputs.  The files hold inputs and expected outputs only.
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from af3_kernels_amd.synthetic import CASES, make_inputs  # noqa: E402
from oracle.dpa_numpy import dpa_closed_form, fused_attention_closed_form, glu_closed_form, layernorm_pair_bias_closed_form  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def save(name, q, k, v, mask, bias):
    want = dpa_closed_form(q, k, v, mask, bias).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), q=q, k=k, v=v, mask=mask, bias=bias, expected=want)
    print(name, q.shape, "max|out|", np.abs(want).max())


def main():
    # cfg1: the CPU-runnable plumbing case, fp32, seed 0
    q, k, v, mask, bias = [t.numpy() for t in make_inputs(CASES["cfg1"])]
    save("cfg1_fp32", q, k, v, mask, bias)
    # small edge cases (values rounded to bf16 so the same file serves the bf16 kernels)
    rng = np.random.default_rng(2024)

    def bf(x):
        return torch.from_numpy(x.astype(np.float32)).to(torch.bfloat16).float().numpy()

    def case(B, H, L, D, mask):
        q, k, v = [bf(rng.standard_normal((B, H, L, D))) for _ in range(3)]
        bias = bf(rng.standard_normal((H, L, L)))
        return q, k, v, mask, bias

    m = np.ones((3, 37), bool); m[1, 20:] = False; m[2, :] = False          # ragged length, one fully dropped row
    save("edge_L37_D32_fullmask", *case(3, 4, 37, 32, m))
    m = np.ones(100, bool); m[90:] = False                                   # 1-D mask, head_dim 24
    save("edge_L100_D24_mask1d", *case(2, 4, 100, 24, m))
    m = np.zeros((2, 70), bool); m[0, 69] = True; m[1, 0] = True             # a single live key per row
    save("edge_L70_D48_onekey", *case(2, 2, 70, 48, m))
    m = rng.random((2, 200)) < 0.5; m[:, 0] = True                          # random mask, head_dim 16
    save("edge_L200_D16_random", *case(1, 2, 200, 16, m[:1]))

    # ---- the fused callers and the ops around them (inputs rounded to bf16; expected values from the float64 numpy forms) ----
    def w(c_in, c_out):
        return bf(rng.standard_normal((c_in, c_out)) / np.sqrt(c_in))

    B, N, C, head = 3, 40, 128, 4                                            # grid self-attention in AlphaFold 3's channel layout
    x, bias = bf(rng.standard_normal((B, N, C))), bf(rng.standard_normal((head, N, N)))
    m = rng.random((B, N)) < 0.8; m[:, 0] = True; m[2, :] = False            # one batch row without any live key
    ws = [w(C, C) for _ in range(5)]
    want = fused_attention_closed_form(x, m, bias, *ws, None, head).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "grid_attention_B3_N40_C128.npz"), x=x, mask=m, bias=bias, wq=ws[0], wk=ws[1], wv=ws[2], wg=ws[3], wo=ws[4], head=head, expected=want)
    print("grid_attention", want.shape, "max|out|", np.abs(want).max())
    N, C, head = 50, 96, 4                                                    # diffusion self-attention: no batch axis, q bias, no output projection
    x, bias, qb = bf(rng.standard_normal((N, C))), bf(rng.standard_normal((head, N, N))), bf(rng.standard_normal(C))
    m = np.ones(N, bool); m[44:] = False
    ws = [w(C, C) for _ in range(4)]
    want = fused_attention_closed_form(x, m, bias, *ws, None, qb, head).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "self_attention_N50_C96.npz"), x=x, mask=m, bias=bias, wq=ws[0], wk=ws[1], wv=ws[2], wg=ws[3], q_bias=qb, head=head, expected=want)
    print("self_attention", want.shape, "max|out|", np.abs(want).max())
    pair = bf(rng.standard_normal((6, 9, 128)) * 2.0 + 1.5)                   # LayerNorm + pair-bias projection
    gamma, beta, wb = bf(1.0 + 0.2 * rng.standard_normal(128)), bf(0.1 * rng.standard_normal(128)), bf(rng.standard_normal((4, 128)) / np.sqrt(128))
    normed, pb = layernorm_pair_bias_closed_form(pair, gamma, beta, wb)
    np.savez_compressed(os.path.join(HERE, "layernorm_pair_bias_6x9x128.npz"), pair=pair, gamma=gamma, beta=beta, wb=wb, eps=1e-5, normed=normed.astype(np.float32), bias=pb.astype(np.float32))
    print("layernorm_pair_bias", normed.shape, pb.shape)
    xg, wg = bf(rng.standard_normal((7, 10, 128))), w(128, 128)               # gated linear unit, 64 output channels
    want = glu_closed_form(xg, wg).astype(np.float32)
    np.savez_compressed(os.path.join(HERE, "glu_70x128_N64.npz"), x=xg, weight=wg, expected=want)
    print("glu", want.shape, "max|out|", np.abs(want).max())


if __name__ == "__main__":
    main()
