"""Import alias so that code written against the reference package name runs unchanged:
`import af3_kernels; from af3_kernels import dot_product_attention_cpp`.  Everything comes from
af3_kernels_amd (the MI355X implementation): the attention hot path, its fused callers (grid and diffusion
self-attention, GridSelfAttentionCpp), the gated linear unit, Linear and the layout helpers."""
from af3_kernels_amd import *  # noqa: F401,F403
from af3_kernels_amd import __all__  # noqa: F401
