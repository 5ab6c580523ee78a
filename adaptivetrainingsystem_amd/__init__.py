"""MI355X (gfx950) native implementation of the sparse-layer path: RMSNorm,
RoPE (GQA), MoE routing / capacity dispatch / SwiGLU experts / combine and
Mixture-of-Depths helpers, as hand-written HIP kernels behind a C ABI
(libats_gfx950.so), with PyTorch modules that keep the reference's names.

Nothing is compiled or loaded at import; the library is loaded on first use and
its absence is an error (there is no fallback path).
"""
from ._lib import AtsError, LIB_PATH, is_built  # noqa: F401
from .layers import (  # noqa: F401
    CapacityMoEFFNLayer,
    DenseGroupedQueryAttention,
    DenseSwiGLU,
    DenseSwiGLUWithMoD,
    FusedRMSNorm,
    FusedRoPE,
    GroupedQueryAttention,
    MoDMoEBlock,
    MoDRouter,
    MoECUDAOps,
    MoEFFNLayer,
    RMSNorm,
    RotaryEmbedding,
    SwiGLUExpert,
    TransformerBlock,
    apply_rotary_pos_emb,
)

__version__ = "0.1.0"
