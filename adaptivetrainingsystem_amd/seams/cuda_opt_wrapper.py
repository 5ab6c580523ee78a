"""Import seam `cuda_opt_wrapper`.

The reference model does
    from cuda_opt_wrapper import FusedRMSNorm, FusedRoPE, FusedSwiGLU, TRANSFORMER_OPS_AVAILABLE
(Src/Main_Scripts/core/model.py:57-68).  Putting this directory on sys.path (or
copying this file over the reference's cuda_opt_wrapper.py) makes those names
resolve to the gfx950 kernels.
"""
import torch
import torch.nn as nn

from adaptivetrainingsystem_amd import _lib, ops
from adaptivetrainingsystem_amd.autograd import SwiGLUFunction
from adaptivetrainingsystem_amd.layers import FusedRMSNorm, FusedRoPE  # noqa: F401

TRANSFORMER_OPS_AVAILABLE = _lib.is_built()


class FusedSwiGLU(nn.Module):
    """Dense-FFN activation block of the reference (cuda_opt_wrapper.py:428-478): two Linear
    projections followed by gate * silu(up); the elementwise part runs in the HIP kernel."""

    def __init__(self, hidden_size: int, intermediate_size: int, use_bias: bool = False):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.use_bias = use_bias
        self.cuda_enabled = True
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=use_bias)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=use_bias)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        gate, up = self.gate_proj(x), self.up_proj(x)
        if torch.is_grad_enabled() and (gate.requires_grad or up.requires_grad):
            return SwiGLUFunction.apply(gate, up)
        return ops.swiglu_mul(gate, up)
