"""FusedLoss and FusedGradClip with the reference's call signatures
(Src/Main_Scripts/training/cuda_kernels.py:91-390), backed by the gfx950 kernels of csrc/train_ops.hip.

Differences that are deliberate: no PyTorch/CPU fallback; results stay on the device (no .item(), no
torch.cuda.synchronize()) except where the reference's interface returns a Python float; the loss
carries a real autograd graph (the reference's fused branch returns a fresh leaf tensor, so nothing
trains through it); per-token weights and bf16 logits / gradients are handled by the kernels.
"""
from __future__ import annotations

from typing import Dict, Iterable, Optional

import torch
from torch.autograd import Function

from . import _lib
from ._lib import ATS_BF16, ATS_F32, AtsError, check

_DT = {torch.float32: ATS_F32, torch.bfloat16: ATS_BF16}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class CrossEntropyFunction(Function):
    """loss = sum_t w_t * ce_t / max(sum_t w_t, 1e-8) over the valid tokens; also saves the statistics."""

    @staticmethod
    def forward(ctx, logits, labels, weights, pad_id, stats):
        T, V = logits.shape
        dev = logits.device
        f32 = dict(dtype=torch.float32, device=dev)
        loss_tok, lse = torch.empty(T, **f32), torch.empty(T, **f32)
        correct, valid = torch.empty(T, **f32), torch.empty(T, **f32)
        sums = torch.empty(5, **f32)
        check(_lib.load().ats_cross_entropy_fwd(logits.data_ptr(), labels.data_ptr(), int(pad_id),
                                                None if weights is None else weights.data_ptr(), loss_tok.data_ptr(),
                                                lse.data_ptr(), correct.data_ptr(), valid.data_ptr(), sums.data_ptr(),
                                                T, V, _DT[logits.dtype], _stream()), "ats_cross_entropy_fwd")
        ctx.save_for_backward(logits, labels, lse, valid, sums, weights if weights is not None else sums.new_empty(0))
        ctx.has_weights = weights is not None
        stats["sums"] = sums
        stats["loss_tok"] = loss_tok
        return sums[0] / torch.clamp(sums[1], min=1e-8)

    @staticmethod
    def backward(ctx, dloss):
        logits, labels, lse, valid, sums, weights = ctx.saved_tensors
        T, V = logits.shape
        dlogits = torch.empty_like(logits)
        scale = dloss.detach().float().reshape(1).contiguous()
        check(_lib.load().ats_cross_entropy_bwd(logits.data_ptr(), labels.data_ptr(), lse.data_ptr(), valid.data_ptr(),
                                                weights.data_ptr() if ctx.has_weights else None, sums.data_ptr(),
                                                scale.data_ptr(), dlogits.data_ptr(), T, V, _DT[logits.dtype],
                                                _stream()), "ats_cross_entropy_bwd")
        return dlogits, None, None, None, None


class FusedLoss:
    """Cross-entropy + accuracy in one pass over the logits.  __call__(logits, labels, loss_weights=None,
    pad_token_id=-100) -> dict(loss, raw_loss, perplexity, valid_tokens, accuracy), all device tensors."""

    def __init__(self):
        self.enabled = _lib.is_built()

    def __call__(self, logits: torch.Tensor, labels: torch.Tensor, loss_weights: Optional[torch.Tensor] = None,
                 pad_token_id: int = -100) -> Dict[str, torch.Tensor]:
        if not logits.is_cuda or not labels.is_cuda:
            raise AtsError("FusedLoss: tensors must be on the GPU (no CPU fallback)")
        if logits.dtype not in _DT:
            raise AtsError(f"FusedLoss: logits dtype {logits.dtype} (float32 or bfloat16)")
        V = logits.shape[-1]
        lg = logits.reshape(-1, V)
        if not lg.is_contiguous():
            lg = lg.contiguous()
        lb = labels.reshape(-1).to(torch.int64).contiguous()
        if lb.numel() != lg.shape[0]:
            raise AtsError(f"FusedLoss: {lg.shape[0]} rows of logits but {lb.numel()} labels")
        w = None
        if loss_weights is not None:
            w = loss_weights.reshape(-1).to(torch.float32).contiguous()
            if w.numel() != lb.numel():
                raise AtsError("FusedLoss: loss_weights must have one entry per token")
        stats: Dict[str, torch.Tensor] = {}
        loss = CrossEntropyFunction.apply(lg, lb, w, int(pad_token_id), stats)
        sums = stats["sums"]
        n_valid = sums[4]
        denom = torch.clamp(n_valid, min=1.0)
        raw = sums[2] / denom                                  # unweighted mean over the valid tokens
        any_valid = n_valid > 0
        inf = torch.full_like(raw, float("inf"))
        return {
            "loss": loss,
            "raw_loss": raw.detach(),
            "perplexity": torch.where(any_valid, torch.exp(torch.clamp(raw.detach(), min=0.0, max=15.0)), inf),
            "valid_tokens": n_valid.detach(),
            "accuracy": (sums[3] / denom).detach(),
        }


class FusedGradClip:
    """Global L2 norm of all gradients and in-place clipping, a fixed number of kernel launches however
    many tensors there are.  __call__(parameters, max_norm) returns the norm as a Python float (the
    reference's interface); norm_and_clip(...) returns it as a device tensor without synchronising."""

    def __init__(self):
        self.cuda_enabled = _lib.is_built()
        self.use_cuda_threshold = 0
        self.total_params = None
        self.implementation = "hip"

    def norm_and_clip(self, parameters: Iterable, max_norm: float, clip: bool = True) -> torch.Tensor:
        # accepts parameters (their .grad is used) or gradient tensors
        grads = [p.grad if isinstance(p, torch.nn.Parameter) else p for p in parameters]
        grads = [g for g in grads if g is not None]
        if not grads:
            return torch.zeros((), dtype=torch.float32, device="cuda")
        dev = grads[0].device
        lib = _lib.load()
        chunk = lib.ats_grad_clip_chunk_elems()
        groups = {}
        for g in grads:
            if not g.is_cuda:
                raise AtsError("FusedGradClip: gradients must be on the GPU (no CPU fallback)")
            if g.dtype not in _DT:
                raise AtsError(f"FusedGradClip: gradient dtype {g.dtype} (float32 or bfloat16)")
            if not g.is_contiguous():
                raise AtsError("FusedGradClip: gradients must be contiguous (they are scaled in place)")
            if g.numel():
                groups.setdefault(g.dtype, []).append(g)
        self.total_params = sum(g.numel() for g in grads)
        norm_out = torch.zeros(2, dtype=torch.float32, device=dev)
        tables = []
        extra = None
        for dtype, gs in groups.items():
            sizes = [g.numel() for g in gs]
            starts = [0]
            for n in sizes:
                starts.append(starts[-1] + (n + chunk - 1) // chunk)
            ptrs = torch.tensor([g.data_ptr() for g in gs], dtype=torch.int64, device=dev)
            sizes_t = torch.tensor(sizes, dtype=torch.int64, device=dev)
            starts_t = torch.tensor(starts, dtype=torch.int32, device=dev)
            partial = torch.empty(max(starts[-1], 1), dtype=torch.float32, device=dev)
            out = torch.zeros(2, dtype=torch.float32, device=dev)
            single = len(groups) == 1
            check(lib.ats_grad_norm_clip(ptrs.data_ptr(), sizes_t.data_ptr(), starts_t.data_ptr(), len(gs), starts[-1],
                                         _DT[dtype], None if extra is None else extra[1:].data_ptr(),
                                         partial.data_ptr(), out.data_ptr(), float(max_norm),
                                         1 if (clip and single) else 0, _stream()), "ats_grad_norm_clip")
            tables.append((ptrs, sizes_t, starts_t, len(gs), starts[-1], dtype, partial))
            extra = out
            norm_out = out
        if clip and len(groups) > 1:      # the norm over all groups is known only now
            for ptrs, sizes_t, starts_t, n, n_chunks, dtype, partial in tables:
                check(lib.ats_grad_norm_clip(ptrs.data_ptr(), sizes_t.data_ptr(), starts_t.data_ptr(), n, n_chunks,
                                             _DT[dtype], None, partial.data_ptr(), norm_out.data_ptr(), float(max_norm),
                                             2, _stream()), "ats_grad_norm_clip")
        return norm_out[0]

    def __call__(self, parameters, max_norm) -> float:
        params = [p for p in parameters]
        return float(self.norm_and_clip([p.grad for p in params if p.grad is not None], max_norm).item())

    def set_implementation(self, mode: str) -> None:
        if mode not in ("auto", "cuda", "hip"):
            raise ValueError(f"Invalid mode '{mode}': this build has one implementation (the HIP kernels)")
        self.implementation = "hip"

    def set_threshold(self, num_params: int) -> None:
        self.use_cuda_threshold = num_params

    def get_info(self):
        return {"cuda_available": self.cuda_enabled, "implementation_mode": self.implementation,
                "cuda_threshold": self.use_cuda_threshold, "total_params": self.total_params, "will_use_cuda": True}
