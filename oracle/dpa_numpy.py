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


# ---- the fused callers and the ops around them, float64 numpy (pins for the C oracle and source of golden vectors) ----
def fused_attention_closed_form(x, mask, bias, wq, wk, wv, wg, wo=None, qbias=None, head=4):
    """examples/grid_self_attention.py:73-92 (after LayerNorm and bias projection) and examples/self_attention.py:64-96:
    x [B, N, C] (or [N, C]); weights are weight^T [C_in, C_out]; returns [B, N, C] (or [N, C])."""
    x = np.asarray(x, np.float64)
    squeeze = x.ndim == 2
    if squeeze:
        x = x[None]
    B, N, C = x.shape
    K = C // head
    split = lambda y: y.reshape(B, N, head, K).transpose(0, 2, 1, 3)
    q = x @ np.asarray(wq, np.float64)
    if qbias is not None:
        q = q + np.asarray(qbias, np.float64).reshape(C)
    core = dpa_closed_form(split(q), split(x @ np.asarray(wk, np.float64)), split(x @ np.asarray(wv, np.float64)), mask, bias)
    out = core.transpose(0, 2, 1, 3).reshape(B, N, C) / (1.0 + np.exp(-(x @ np.asarray(wg, np.float64))))
    if wo is not None:
        out = out @ np.asarray(wo, np.float64)
    return out[0] if squeeze else out


def layernorm_pair_bias_closed_form(pair, gamma, beta, wb, eps=1e-5):
    """src/af3_kernels/Attention.py:51-52: LayerNorm over the last axis, then bias[h] = normed . wb[h]; returns (normed, bias [H, ...])."""
    x = np.asarray(pair, np.float64)
    mean = x.mean(-1, keepdims=True)
    var = ((x - mean) ** 2).mean(-1, keepdims=True)
    normed = (x - mean) / np.sqrt(var + eps) * np.asarray(gamma, np.float64) + np.asarray(beta, np.float64)
    bias = np.moveaxis(normed @ np.asarray(wb, np.float64).T, -1, 0)
    return normed, bias


def glu_closed_form(x, weight):
    """examples/gated_linear_unit.py:18-22."""
    y = np.asarray(x, np.float64) @ np.asarray(weight, np.float64)
    n = y.shape[-1] // 2
    a, b = y[..., :n], y[..., n:]
    return a / (1.0 + np.exp(-a)) * b
