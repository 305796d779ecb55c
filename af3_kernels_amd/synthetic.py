"""Seeded synthetic inputs for the five benchmark cases of the biased-attention path.

Shapes follow the shapes the reference's harness runs (examples/dot_product_attention.py:47-85:
`(L,4,L,32)` triangle attention, `(1,16,L,24|48)` diffusion attention); values are drawn in
fp32 from one torch CPU generator in the order q, k, v, bias and then cast, so a case is
reproducible from its name and seed alone.  Masks: truthy = attend.
"""
from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class Case:
    name: str
    B: int
    H: int
    L: int
    D: int
    io_dtype: str          # "fp32" | "bf16"
    mma_dtype: str         # "fp32" | "bf16" | "fp8"
    mask_kind: str         # "tail:<n>" (last n keys dropped), "tail1:<n>" (only in the last batch row), "bernoulli:<keep>"
    mask_rank: int         # 1 -> [L], 2 -> [B,L]
    tol: float             # max-abs tolerance against the fp32 formula
    seed: int = 0

    @property
    def flops(self) -> float:
        return 4.0 * self.B * self.H * self.L * self.L * self.D

    @property
    def bytes(self) -> float:
        io = 4 if self.io_dtype == "fp32" else 2
        bias = 4 if self.io_dtype == "fp32" else 2
        return 4.0 * self.B * self.H * self.L * self.D * io + self.H * self.L * self.L * bias + self.B * self.L


CASES = {
    # CPU-runnable plumbing case
    "cfg1": Case("cfg1", 2, 4, 128, 32, "fp32", "fp32", "tail1:16", 2, 1e-4),
    # AF3 triangle attention, N=384
    "cfg2": Case("cfg2", 384, 4, 384, 32, "bf16", "bf16", "tail:38", 2, 2e-2),
    # pairformer single attention with pair bias, N=768, 16 heads x 24
    "cfg3": Case("cfg3", 1, 16, 768, 24, "bf16", "bf16", "tail:38", 1, 2e-2),
    # large-crop triangle attention, N=768 (headline)
    "cfg4": Case("cfg4", 768, 4, 768, 32, "bf16", "bf16", "bernoulli:0.92", 2, 2e-2),
    # diffusion transformer token attention, fp8 MMA with bf16 I/O
    "cfg5": Case("cfg5", 5, 16, 1536, 24, "bf16", "fp8", "tail:154", 1, 6e-2),
    # not one of the named configurations: a triangle-attention slab in float32, sized to measure the fp32 matrix-core kernel
    "fp32_n768": Case("fp32_n768", 64, 4, 768, 32, "fp32", "fp32", "bernoulli:0.92", 2, 1e-4),
}


def make_mask(case: Case, gen: torch.Generator) -> torch.Tensor:
    kind, _, arg = case.mask_kind.partition(":")
    B, L = case.B, case.L
    if kind == "tail":
        m = torch.ones(L, dtype=torch.bool)
        m[L - int(arg):] = False
        return m if case.mask_rank == 1 else m[None, :].expand(B, L).contiguous()
    if kind == "tail1":
        m = torch.ones(B, L, dtype=torch.bool)
        m[B - 1, L - int(arg):] = False
        return m
    if kind == "bernoulli":
        m = torch.rand(B, L, generator=gen) < float(arg)
        m[:, 0] |= ~m.any(dim=1)  # at least one live key per row
        return m
    raise ValueError(case.mask_kind)


def make_inputs(case, device="cpu", batch=None):
    """Returns q, k, v, mask, bias.  `batch` truncates the batch axis (a bounded sample of the
    same workload: the bias and per-row work are unchanged)."""
    if isinstance(case, str):
        case = CASES[case]
    gen = torch.Generator(device="cpu")
    gen.manual_seed(case.seed)
    B = case.B if batch is None else min(batch, case.B)
    dt = torch.float32 if case.io_dtype == "fp32" else torch.bfloat16
    shape = (B, case.H, case.L, case.D)

    def draw(s):
        return torch.randn(s, generator=gen, dtype=torch.float32)

    q, k, v = draw(shape), draw(shape), draw(shape)
    bias = draw((case.H, case.L, case.L))
    mgen = torch.Generator(device="cpu")
    mgen.manual_seed(case.seed + 1)
    mask = make_mask(case, mgen)
    if mask.dim() == 2:
        mask = mask[:B]
    q, k, v, bias = [t.to(dt).to(device) for t in (q, k, v, bias)]
    return q, k, v, mask.to(device), bias


# ------------------------------------------------------------------------------------------
# the fused callers of the attention core (shapes of examples/grid_self_attention.py:141-167 and
# examples/self_attention.py: pair [N, N, 128] with 4 heads; tokens [N, 768] with 16 heads)
# ------------------------------------------------------------------------------------------
@dataclass(frozen=True)
class FusedCase:
    name: str
    kind: str              # "grid" (_attention_cpp) | "self" (self_attention_cpp)
    B: int                 # batch rows (grid: = N; self: 1)
    N: int
    C: int
    head: int
    keep: float = 0.92     # Bernoulli key mask
    seed: int = 0

    @property
    def flops_projections(self) -> float:
        return 2.0 * self.B * self.N * self.C * 4 * self.C

    @property
    def flops_attention(self) -> float:
        return 4.0 * self.B * self.N * self.N * self.C

    @property
    def flops_out_projection(self) -> float:
        return 2.0 * self.B * self.N * self.C * self.C if self.kind == "grid" else 0.0

    @property
    def flops(self) -> float:
        return self.flops_projections + self.flops_attention + self.flops_out_projection

    @property
    def bytes(self) -> float:
        """Algorithmic bytes of the whole op: rows in, rows out, bias, mask, weights (bf16)."""
        return 2.0 * (2 * self.B * self.N * self.C + self.head * self.N * self.N + 5 * self.C * self.C) + self.B * self.N


FUSED_CASES = {
    "grid_n384": FusedCase("grid_n384", "grid", 384, 384, 128, 4),
    "grid_n768": FusedCase("grid_n768", "grid", 768, 768, 128, 4),
    # the reference harness's default set (examples/grid_self_attention.py:161-169): K and V of a head no longer fit in LDS,
    # so this one runs as projection GEMM + attention kernel + output GEMM
    "grid_n1536": FusedCase("grid_n1536", "grid", 1536, 1536, 128, 4),
    "self_n1536": FusedCase("self_n1536", "self", 1, 1536, 768, 16),
    # five diffusion samples of the same tokens in one call (16 heads of 24 channels: the shape of cfg5, in bf16): the samples share every bias tile
    "self5_n1536": FusedCase("self5_n1536", "self", 5, 1536, 384, 16),
}


def make_fused_inputs(case, device="cpu", batch=None):
    """Returns dict(x, mask, bias, wq, wk, wv, wg, wo, q_bias) of bfloat16 tensors; the weights are weight^T in
    natural [C_in, C_out] layout, scaled by C^-1/2 so that projected rows have unit scale.  `batch` truncates the
    batch axis of a grid case."""
    if isinstance(case, str):
        case = FUSED_CASES[case]
    gen = torch.Generator(device="cpu")
    gen.manual_seed(case.seed)
    B = case.B if batch is None else min(batch, case.B)
    dt = torch.bfloat16
    draw = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    ws = [(draw(case.C, case.C) * case.C ** -0.5).to(dt).to(device) for _ in range(5)]
    bias = draw(case.head, case.N, case.N).to(dt).to(device)
    q_bias = draw(case.C).to(dt).to(device)
    mgen = torch.Generator(device="cpu")
    mgen.manual_seed(case.seed + 1)
    if case.kind == "grid":
        mask = torch.rand(case.B, case.N, generator=mgen) < case.keep
        mask[:, 0] = True
        mask = mask[:B]
        # (rows are drawn per batch row so that a truncated sample sees the same leading rows)
        x = torch.stack([draw(case.N, case.C) for _ in range(B)]).to(dt).to(device)
    else:
        mask = torch.rand(case.N, generator=mgen) < case.keep
        mask[0] = True
        x = (draw(case.N, case.C) if case.B == 1 else torch.stack([draw(case.N, case.C) for _ in range(B)])).to(dt).to(device)
    return dict(x=x, mask=mask.to(device), bias=bias, wq=ws[0], wk=ws[1], wv=ws[2], wg=ws[3], wo=ws[4] if case.kind == "grid" else None,
                q_bias=q_bias if case.kind == "self" else None)
