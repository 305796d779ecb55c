"""Independent float64 statements of the attention formula (TEST INFRASTRUCTURE ONLY).

`dpa_closed_form` is the vectorised numpy form of examples/dot_product_attention.py:20-43;
`dpa_brute_force` is the same thing as scalar Python loops for tiny shapes.  They exist to
pin oracle/af3_oracle.c, which is what the GPU kernels are compared with.
"""
import math

import numpy as np


def lift_mask(mask, B, L):
    m = np.asarray(mask).astype(bool)
    if m.ndim == 1:  # examples/dot_product_attention.py:34-35
        m = np.broadcast_to(m[None, :], (B, L))
    return m.reshape(B, L)


def dpa_closed_form(q, k, v, mask, bias):
    q = np.asarray(q, np.float64); k = np.asarray(k, np.float64); v = np.asarray(v, np.float64)
    B, H, L, D = q.shape
    logits = np.einsum("bhqd,bhkd->bhqk", q * D ** -0.5, k)
    if bias is not None:
        logits = logits + np.asarray(bias, np.float64)[None]
    if mask is not None:
        keep = lift_mask(mask, B, L)
        logits = np.where(keep[:, None, None, :], logits, -1e9)
    logits = logits - logits.max(-1, keepdims=True)
    w = np.exp(logits)
    w /= w.sum(-1, keepdims=True)
    return np.einsum("bhqk,bhkd->bhqd", w, v)


def dpa_brute_force(q, k, v, mask, bias):
    B, H, L, D = q.shape
    keep = lift_mask(mask, B, L)
    out = np.zeros((B, H, L, D))
    for b in range(B):
        for h in range(H):
            for i in range(L):
                s = []
                for j in range(L):
                    acc = 0.0
                    for d in range(D):
                        acc += float(q[b, h, i, d]) / math.sqrt(D) * float(k[b, h, j, d])
                    acc += float(bias[h, i, j])
                    if not keep[b, j]:
                        acc = -1e9
                    s.append(acc)
                mx = max(s)
                e = [math.exp(x - mx) for x in s]
                z = sum(e)
                for d in range(D):
                    out[b, h, i, d] = sum(e[j] * float(v[b, h, j, d]) for j in range(L)) / z
    return out
