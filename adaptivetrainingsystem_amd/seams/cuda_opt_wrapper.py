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
from adaptivetrainingsystem_amd.autograd import LinearFunction, SwiGLUFunction
from adaptivetrainingsystem_amd.layers import FusedRMSNorm, FusedRoPE, _as_dtype, _wants_grad  # noqa: F401

TRANSFORMER_OPS_AVAILABLE = _lib.is_built()


class FusedSwiGLU(nn.Module):
    """Dense-FFN activation block of the reference (cuda_opt_wrapper.py:428-478): two Linear projections
    followed by gate * silu(up).  The parameters are the reference's (gate_proj, up_proj), so state_dicts
    load unchanged; the arithmetic runs in the HIP kernels:

    * inference without biases: one GEMM over the stacked [up_proj; gate_proj] weight whose epilogue applies
      silu(first half) * second half, so neither projection is written to memory (K-sliced for a few rows);
    * with autograd, or with biases: the two projections through the single-group GEMM (forward, dgrad and
      wgrad), then the elementwise kernel and its backward."""

    def __init__(self, hidden_size: int, intermediate_size: int, use_bias: bool = False):
        super().__init__()
        self.hidden_size = hidden_size
        self.intermediate_size = intermediate_size
        self.use_bias = use_bias
        self.cuda_enabled = True
        self.gate_proj = nn.Linear(hidden_size, intermediate_size, bias=use_bias)
        self.up_proj = nn.Linear(hidden_size, intermediate_size, bias=use_bias)
        self._state = {"key": None, "w": None}      # plain dict: not a buffer, not in the state_dict

    def _stacked_up_gate(self, dtype: torch.dtype) -> torch.Tensor:
        """[up_proj; gate_proj] as one [2I, H] matrix in the compute dtype, rebuilt when a weight is replaced or
        written to (version counters; a write through `weight.data` needs reset_cached_weights())."""
        ws = (self.up_proj.weight, self.gate_proj.weight)
        key = (dtype,) + tuple((w.data_ptr(), w._version) for w in ws)
        st = self._state
        if st["key"] != key:
            with torch.no_grad():
                st["w"] = torch.cat([w.detach().to(dtype) for w in ws], dim=0).contiguous()
            st["key"] = key
        return st["w"]

    def reset_cached_weights(self) -> None:
        self._state["key"] = None
        self._state["w"] = None

    def _project(self, x2: torch.Tensor, lin: nn.Linear, grad: bool) -> torch.Tensor:
        y = LinearFunction.apply(x2, lin.weight) if grad else ops.linear_nt(x2, _as_dtype(lin.weight, x2.dtype))
        return y if lin.bias is None else y + lin.bias.to(y.dtype)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        H, I = self.hidden_size, self.intermediate_size
        if x.shape[-1] != H:
            raise _lib.AtsError(f"FusedSwiGLU: last dimension {x.shape[-1]} != hidden_size {H}")
        if x.dtype == torch.float16:
            # as the reference's wrapper serves every dtype (cuda_opt_wrapper.py:217): up-cast, float32 kernels,
            # one rounding back; inference only (the matrices would need float32 master copies to train)
            if _wants_grad(x, *self.parameters()):
                raise _lib.AtsError("FusedSwiGLU: float16 activations are served through the float32 kernels for "
                                    "inference only; train in bfloat16 or float32")
            return self.forward(x.float()).to(x.dtype)
        out_shape = x.shape[:-1] + (I,)
        x2 = x.reshape(-1, H).contiguous()
        n = x2.shape[0]
        if n == 0:
            return x.new_empty(out_shape)
        grad = _wants_grad(x, *self.parameters())
        if grad or self.use_bias:
            gate, up = self._project(x2, self.gate_proj, grad), self._project(x2, self.up_proj, grad)
            h = SwiGLUFunction.apply(gate, up) if grad else ops.swiglu_mul(gate, up)
            return h.view(out_shape)
        w = self._stacked_up_gate(x2.dtype)
        start = torch.zeros(1, dtype=torch.int32, device=x.device)
        count = torch.full((1,), n, dtype=torch.int32, device=x.device)
        splits = ops.down_k_splits(1, n, 2 * I, H, x2.dtype) if I % 8 == 0 and n <= 32 else 1
        if splits > 1:
            h = ops.swiglu_partials(ops.grouped_down_splitk(x2, ops.weight_pointer_table([w]), start, count, n,
                                                            2 * I, H, splits), x2.dtype)
        else:
            h = ops.grouped_gateup_swiglu(x2, ops.weight_pointer_table([w]), start, count, n, n, H, I)
        return h.view(out_shape)
