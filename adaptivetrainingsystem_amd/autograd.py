"""Autograd functions over the gfx950 kernels, so that a transformer block trains through the HIP
path.  Every forward and backward step is a kernel of libats_gfx950; torch is used for tensor
allocation, a handful of E-element scalar expressions and the autograd graph itself.

Reference counterparts (MS = Src/Main_Scripts of the reference checkout):
  RMSNormFunction / RoPEFunction / SwiGLUFunction   MS/core/cuda_opt_wrapper.py:85-254
  MoE layer: the reference trains it through plain PyTorch autograd over MS/core/model.py:1160-1263
  (noise on the routing logits in training mode, model.py:1203-1205; the auxiliary loss is taken on
  the noise-free logits with the usage histogram as a constant, model.py:1190-1192, 1244-1263).
"""
from __future__ import annotations

from typing import Optional

import torch
from torch.autograd import Function

from . import ops
from ._lib import ROUTE_SOFTMAX_TOPK, ROUTE_TOPK_SOFTMAX


def _grad_to(g: Optional[torch.Tensor], like: torch.Tensor) -> Optional[torch.Tensor]:
    if g is None:
        return None
    return g if g.dtype == like.dtype else g.to(like.dtype)


class RMSNormFunction(Function):
    @staticmethod
    def forward(ctx, x, weight, eps):
        ctx.save_for_backward(x, weight)
        ctx.eps = eps
        return ops.rmsnorm(x, weight, eps)

    @staticmethod
    def backward(ctx, dy):
        x, weight = ctx.saved_tensors
        need_dw = weight is not None and ctx.needs_input_grad[1]
        dx, dw = ops.rmsnorm_bwd(x, weight, dy.to(x.dtype), ctx.eps, need_dw=need_dw)
        return dx, (_grad_to(dw, weight) if need_dw else None), None


class RoPEFunction(Function):
    @staticmethod
    def forward(ctx, q, k, cos, sin, position_offset):
        ctx.save_for_backward(cos, sin)
        ctx.position_offset = position_offset
        q_out, k_out = ops.rope(q, k, cos, sin, position_offset)
        return q_out, k_out

    @staticmethod
    def backward(ctx, dq, dk):
        cos, sin = ctx.saved_tensors
        gq, gk = ops.rope(dq, dk, cos, sin, ctx.position_offset, inverse=True)
        return gq, gk, None, None, None


class GatherRowsFunction(Function):
    """out[i] = x[rows[i]] for x [N, H] and distinct int32 rows; the gradient is the scatter-add of the
    cotangent rows onto zeros (every other row of x gets none)."""

    @staticmethod
    def forward(ctx, x, rows):
        ctx.save_for_backward(rows)
        ctx.n = x.shape[0]
        return ops.gather_rows(x.contiguous(), rows)

    @staticmethod
    def backward(ctx, dout):
        (rows,) = ctx.saved_tensors
        dx = torch.zeros(ctx.n, dout.shape[1], dtype=dout.dtype, device=dout.device)
        ops.scatter_add_rows(dx, rows, dout.contiguous())
        return dx, None


class ScatterAddRowsFunction(Function):
    """out = x with out[rows[i]] += delta[i] (distinct rows), out of place: the cotangent passes to x
    unchanged and its selected rows are the gradient of delta."""

    @staticmethod
    def forward(ctx, x, rows, delta):
        ctx.save_for_backward(rows)
        out = x.contiguous().clone()
        ops.scatter_add_rows(out, rows, delta.to(out.dtype))
        return out

    @staticmethod
    def backward(ctx, dout):
        (rows,) = ctx.saved_tensors
        return dout, None, ops.gather_rows(dout.contiguous(), rows)


class AttentionFunction(Function):
    """Causal grouped-query attention: q [B,Hq,L,D], k, v [B,Hkv,Lk,D] -> [B, L, Hq*D]; key_bias
    [B, Lk] / pair_bias [B or 1, (Hq or 1,) L, Lk] float32 or None (constants: they get no gradient); dropout_p with the
    seed that the backward reuses."""

    @staticmethod
    def forward(ctx, q, k, v, scale, key_bias=None, pair_bias=None, dropout_p=0.0, dropout_seed=0):
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        out, lse = ops.causal_attention(q, k, v, scale, return_lse=True, key_bias=key_bias, pair_bias=pair_bias,
                                        dropout_p=dropout_p, dropout_seed=dropout_seed)
        ctx.save_for_backward(q, k, v, out, lse, key_bias, pair_bias)
        ctx.scale = scale
        ctx.dropout = (float(dropout_p), int(dropout_seed))
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, key_bias, pair_bias = ctx.saved_tensors
        dq, dk, dv = ops.causal_attention_bwd(q, k, v, out, lse, dout, ctx.scale, key_bias=key_bias,
                                              pair_bias=pair_bias, dropout_p=ctx.dropout[0],
                                              dropout_seed=ctx.dropout[1])
        return dq, dk, dv, None, None, None, None, None


class AttentionF32Function(Function):
    """The float32 route of the attention (ops.attention_f32): same arguments as AttentionFunction; the softmax
    weights are kept for the backward, as autograd keeps them for the reference."""

    @staticmethod
    def forward(ctx, q, k, v, scale, key_bias=None, pair_bias=None, dropout_p=0.0, dropout_seed=0):
        out, state = ops.attention_f32(q, k, v, scale, key_bias=key_bias, pair_bias=pair_bias, dropout_p=dropout_p,
                                       dropout_seed=dropout_seed, return_weights=True)
        w, w_drop, qp, kp, vp = state
        ctx.save_for_backward(w, w_drop, qp, kp, vp)
        ctx.meta = (q.shape[0], q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3], scale, float(dropout_p),
                    int(dropout_seed))
        return out

    @staticmethod
    def backward(ctx, dout):
        B, Hq, Hkv, L, Lk, D, scale, p, seed = ctx.meta
        dq, dk, dv = ops.attention_f32_bwd(ctx.saved_tensors, dout.contiguous(), B, Hq, Hkv, L, Lk, D, scale, p, seed)
        return dq, dk, dv, None, None, None, None, None


class LinearFunction(Function):
    """y = x @ weight^T for x [T, K], weight [N, K] (a bias-free nn.Linear) through the grouped GEMM kernels
    with one group: dgrad reads the weight as it is where the K-major kernel applies (bfloat16, more than 192
    rows) and multiplies by a transposed copy otherwise, wgrad multiplies the transposed activations."""

    @staticmethod
    def forward(ctx, x, weight):
        x = x.contiguous()
        w = weight.detach().to(x.dtype).contiguous()
        ctx.save_for_backward(x, w)
        ctx.param_dtype = weight.dtype
        return ops.linear_nt(x, w)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        T, K = x.shape
        N = w.shape[0]
        dy = dy.to(x.dtype).contiguous()
        dx = dw = None
        offsets = torch.tensor([0, T], dtype=torch.int32, device=x.device)
        kept = offsets[1:].clone()
        if ctx.needs_input_grad[0]:
            if DGRAD_FROM_FORWARD_WEIGHTS and ops.grouped_gemm_nn_supported(1, T, K, N, K, x.dtype):
                dx = ops.grouped_gemm_nn(ops.weight_pointer_table([w]), K, offsets, kept, T, T, K, N, dy)
            else:
                wT, tab = ops.transpose_batched([w])             # [K, N]; kept alive until the GEMM is queued
                dx = ops.grouped_gemm_nt(tab, N, K, offsets, kept, T, T, K, N, a=dy)
        if ctx.needs_input_grad[1]:
            ks, kc = ops.wgrad_plan(kept)
            ld = ops.wgrad_padded_rows(T, 1)
            dyT = ops.transpose_grouped_rows(dy, offsets, kept, T)
            xT = ops.transpose_grouped_rows(x, offsets, kept, T)
            es = x.element_size()
            a_ptrs = ks.long() * es + dyT.data_ptr()
            b_ptrs = ks.long() * es + xT.data_ptr()
            rs = torch.zeros(1, dtype=torch.int32, device=x.device)
            rc = torch.full((1,), N, dtype=torch.int32, device=x.device)
            dw = ops.grouped_gemm_nt(b_ptrs, ld, K, rs, rc, N, N, K, ld, a_ptrs=a_ptrs, lda=ld, k_count=kc,
                                     dtype=x.dtype, out_dtype=x.dtype).to(ctx.param_dtype)
        return dx, dw


class SwiGLUFunction(Function):
    """out = gate * silu(up) (the dense-FFN convention of the fused wrapper)."""

    @staticmethod
    def forward(ctx, gate, up):
        shape = gate.shape
        g2, u2 = gate.reshape(-1, shape[-1]).contiguous(), up.reshape(-1, shape[-1]).contiguous()
        ctx.save_for_backward(g2, u2)
        ctx.shape = shape
        return ops.silu_mul(u2, g2).view(shape)

    @staticmethod
    def backward(ctx, dout):
        g2, u2 = ctx.saved_tensors
        d2 = dout.reshape(g2.shape).to(g2.dtype).contiguous()
        du, dg = ops.silu_mul_bwd(u2, g2, d2)
        return dg.view(ctx.shape), du.view(ctx.shape)


# Whether the fused bfloat16 training kernels also write the transposed copies of h and dgu that the weight-gradient
# products contract over (otherwise separate transposing passes produce them; same bits either way).
FUSE_TRANSPOSED_COPIES = True
# Data gradients of the expert products read the weights as the forward holds them ([out, in], the reduction
# index along the rows) where the K-major kernel applies (bfloat16, prefill-sized groups), instead of multiplying
# by a transposed copy made per step.
DGRAD_FROM_FORWARD_WEIGHTS = True


def _ffn_forward(x, wgu, wd, offsets, kept, rows, row_src, k, want_wgrad=False):
    """Expert FFN over the grouped rows, keeping the gate/up pre-activations for the backward pass.
    Returns (gu [rows, 2I], h [rows, I], y [rows, H], hT, wplan): with want_wgrad, wplan = the weight-gradient
    layout of these groups (ops.wgrad_plan) and, where the fused bfloat16 kernel runs, hT = h already transposed
    into it by that kernel (the backward pass then keeps hT instead of h); otherwise None."""
    H, I = x.shape[1], wd[0].shape[1]
    tab_gu, tab_d = ops.weight_pointer_table(wgu), ops.weight_pointer_table(wd)
    wplan = ops.wgrad_plan(kept) if want_wgrad and rows > 0 else None
    hT = None
    both = ops.grouped_gateup_swiglu_save(x, tab_gu, offsets, kept, rows, rows, H, I, a_rows=row_src, a_row_div=k,
                                          t_col0=wplan[0] if wplan is not None and FUSE_TRANSPOSED_COPIES else None)
    if both is not None:             # prefill-sized groups: one kernel writes the pre-activations and h
        gu, h, hT = both
    else:
        gu = ops.grouped_gemm_nt(tab_gu, H, 2 * I, offsets, kept, rows, rows, 2 * I, H, a=x, a_rows=row_src,
                                 a_row_div=k)
        h = ops.silu_mul(gu[:, :I], gu[:, I:], rows_dev=offsets[-1:])      # only the kept rows
    y = ops.grouped_down(h, tab_d, offsets, kept, rows, H, I)
    return gu, h, y, hT, wplan


def _ffn_backward(dy, x, wgu, wd, gu, h, offsets, kept, rows, row_src, k, need_x, need_w, hT=None, wplan=None):
    """Gradients of _ffn_forward: dx_rows [rows, H] (or None), dWgu [E, 2I, H], dWd [E, H, I] (or None).
    dgrad multiplies by per-step transposed copies of the weights; wgrad multiplies the transposed,
    zero-padded activations of each expert (K = its padded row count).  h may be None when hT, its transposed
    copy from the forward kernel, is given; the fused bfloat16 dgrad kernel likewise hands back dgu and its
    transposed copy, so only dy and the gathered x go through a transposing pass."""
    E = len(wd)
    H, I = x.shape[1], wd[0].shape[1]
    dtype, dev = x.dtype, x.device
    if need_w and wplan is None:
        wplan = ops.wgrad_plan(kept)
    dguT = None
    t_col0 = wplan[0] if need_w and FUSE_TRANSPOSED_COPIES else None
    if DGRAD_FROM_FORWARD_WEIGHTS and ops.grouped_down_dgrad_dsilu_supported(E, rows, H, I, dtype, transposed_weights=False):
        # prefill-sized bfloat16 groups: one kernel, reading the down weights as the forward holds them
        pair = ops.grouped_down_dgrad_dsilu(dy, ops.weight_pointer_table(list(wd)), gu, offsets, kept, rows, H, I,
                                            t_col0=t_col0, transposed_weights=False)
    else:
        wdT, tab_dT = ops.transpose_batched(wd)                  # [I, H] per expert; kept alive until return
        pair = ops.grouped_down_dgrad_dsilu(dy, tab_dT, gu, offsets, kept, rows, H, I, t_col0=t_col0)   # one kernel
    dgu = None
    if pair is not None:
        dgu, dguT = pair
    if dgu is None:                                              # smaller groups, float32: two kernels
        dh = ops.grouped_gemm_nt(tab_dT, H, I, offsets, kept, rows, rows, I, H, a=dy)
        dgu = torch.empty_like(gu)
        ops.silu_mul_bwd(gu[:, :I], gu[:, I:], dh, da=dgu[:, :I], db=dgu[:, I:], rows_dev=offsets[-1:])
    dx_rows = dwgu = dwd = None
    if need_x:
        if DGRAD_FROM_FORWARD_WEIGHTS and ops.grouped_gemm_nn_supported(E, rows, H, 2 * I, H, dtype):
            dx_rows = ops.grouped_gemm_nn(ops.weight_pointer_table(list(wgu)), H, offsets, kept, rows, rows, H, 2 * I, dgu)
        else:
            wguT, tab_guT = ops.transpose_batched(wgu)           # [H, 2I] per expert
            dx_rows = ops.grouped_gemm_nt(tab_guT, 2 * I, H, offsets, kept, rows, rows, H, 2 * I, a=dgu)
    if need_w:
        ks, kc = wplan
        ld = ops.wgrad_padded_rows(rows, E)
        es = x.element_size()

        def wgrad(lhs, rhs, M, N, gather=None, lhsT=None, rhsT=None):
            if lhsT is None:
                lhsT = ops.transpose_grouped_rows(lhs, offsets, kept, rows)
            if rhsT is None:
                rhsT = ops.transpose_grouped_rows(rhs, offsets, kept, rows, gather=gather, gather_div=k)
            a_ptrs = ks.long() * es + lhsT.data_ptr()
            b_ptrs = ks.long() * es + rhsT.data_ptr()
            rs = torch.arange(E, dtype=torch.int32, device=dev) * M
            rc = torch.full((E,), M, dtype=torch.int32, device=dev)
            g = ops.grouped_gemm_nt(b_ptrs, ld, N, rs, rc, E * M, E * M, N, ld, a_ptrs=a_ptrs, lda=ld, k_count=kc,
                                    dtype=dtype, out_dtype=dtype)
            return g.view(E, M, N)

        dwd = wgrad(dy, h, H, I, rhsT=hT)
        dwgu = wgrad(dgu, x, 2 * I, H, gather=row_src, lhsT=dguT)
    return dx_rows, dwgu, dwd


class ExpertFFNFunction(Function):
    """One SwiGLU expert over every row of x [n, H]: down(silu(gate) * up)."""

    @staticmethod
    def forward(ctx, x, w_gate_up, w_down):
        dtype = x.dtype
        x = x.contiguous()
        wgu, wd = [w_gate_up.detach().to(dtype).contiguous()], [w_down.detach().to(dtype).contiguous()]
        n = x.shape[0]
        offsets = torch.tensor([0, n], dtype=torch.int32, device=x.device)
        kept = offsets[1:].clone()
        gu, h, y, hT, wplan = _ffn_forward(x, wgu, wd, offsets, kept, n, None, 1,
                                           want_wgrad=ctx.needs_input_grad[1] or ctx.needs_input_grad[2])
        ctx.h_transposed = hT is not None
        ctx.has_wplan = wplan is not None
        ctx.save_for_backward(x, offsets, kept, gu, hT if hT is not None else h, *(wplan or ()))
        ctx.wgu, ctx.wd = wgu, wd
        ctx.param_dtypes = (w_gate_up.dtype, w_down.dtype)
        return y

    @staticmethod
    def backward(ctx, dy):
        saved = ctx.saved_tensors                    # read once: activation checkpointing unpacks on every access
        x, offsets, kept, gu, h = saved[:5]
        wplan = tuple(saved[5:7]) if ctx.has_wplan else None
        hT = None
        if ctx.h_transposed:
            h, hT = None, h
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1] or ctx.needs_input_grad[2]
        dx, dwgu, dwd = _ffn_backward(dy.to(x.dtype).contiguous(), x, ctx.wgu, ctx.wd, gu, h, offsets, kept,
                                      x.shape[0], None, 1, need_x, need_w, hT=hT, wplan=wplan)
        return (dx, dwgu[0].to(ctx.param_dtypes[0]) if need_w else None,
                dwd[0].to(ctx.param_dtypes[1]) if need_w else None)


class MoEFunction(Function):
    """The whole MoE FFN layer on [T, H] tokens.  apply(x, gate_weight, cfg, *expert_weights) with
    expert_weights = E gate/up matrices [2I, H] followed by E down matrices [H, I]; cfg is a dict:
    top_k, temperature, variant, capacity (C, or T for no dropping), load_balancing_weight,
    noise_std (0 in eval), logit_bias (tensor or None), stats (dict filled with the plan).
    Returns (out [T, H], aux scalar)."""

    @staticmethod
    def forward(ctx, x, gate_weight, cfg, *expert_weights):
        E = len(expert_weights) // 2
        k, C = cfg["top_k"], cfg["capacity"]
        T, H = x.shape
        dtype = x.dtype
        wg = gate_weight.detach().to(dtype).contiguous()
        wgu = [w.detach().to(dtype).contiguous() for w in expert_weights[:E]]
        wd = [w.detach().to(dtype).contiguous() for w in expert_weights[E:]]
        I = wd[0].shape[1]
        x = x.contiguous()

        logits = ops.router_logits(x, wg, cfg.get("logit_bias"))
        logits_route = logits
        if cfg.get("noise_std", 0.0) > 0:
            logits_route = logits + torch.randn_like(logits) * cfg["noise_std"]
        route = ops.route_topk(logits_route, k, cfg["temperature"], cfg["variant"], cfg["load_balancing_weight"])
        usage = route["hist"].float() / (T * k + 1e-9)
        if logits_route is logits:
            aux = route["aux"][0]
        else:   # importance from the noise-free logits (model.py:1190-1192)
            aux = ops.aux_loss_clean_logits(logits, route["hist"], k, cfg["variant"], cfg["load_balancing_weight"])
        plan = ops.dispatch_plan(route["indices"], E, C)
        rows = min(T * k, E * C)
        hT = wplan = None
        if rows > 0:
            gu, h, y, hT, wplan = _ffn_forward(x, wgu, wd, plan["offsets"], plan["kept"], rows, plan["row_src"], k,
                                               want_wgrad=any(ctx.needs_input_grad[3:]))
        else:
            gu = torch.zeros(1, 2 * I, dtype=dtype, device=x.device)
            h = torch.zeros(1, I, dtype=dtype, device=x.device)
            y = torch.zeros(1, H, dtype=dtype, device=x.device)
        out = ops.combine(y, plan["row_of"], route["weights"], T, k, out_dtype=dtype)

        ctx.cfg = {key: cfg[key] for key in ("top_k", "temperature", "variant", "load_balancing_weight")}
        ctx.dims = (T, H, I, E, rows)
        ctx.n_weights = len(expert_weights)
        ctx.wgu, ctx.wd = wgu, wd          # dtype copies (or the parameters' own storage); not graph tensors
        ctx.h_transposed = hT is not None       # then the kernel's transposed copy of h is kept instead of h
        ctx.has_wplan = wplan is not None
        ctx.save_for_backward(x, wg, logits, logits_route, route["indices"], route["weights"], usage, aux.detach(),
                              plan["offsets"], plan["kept"], plan["row_src"], plan["row_of"], gu,
                              hT if hT is not None else h, y, *(wplan or ()))
        ctx.param_dtypes = (gate_weight.dtype, [w.dtype for w in expert_weights])
        if cfg.get("stats") is not None:
            cfg["stats"].update({"logits": logits, "capacity": C, **route, **plan, "aux": aux.detach().reshape(1)})
        return out, aux

    @staticmethod
    def backward(ctx, dout, daux):
        saved = ctx.saved_tensors                    # read once: activation checkpointing unpacks on every access
        (x, wg, logits, logits_route, idx, w, usage, aux, offsets, kept, row_src, row_of, gu, h, y) = saved[:15]
        wplan = tuple(saved[15:17]) if ctx.has_wplan else None
        hT = None
        if ctx.h_transposed:
            h, hT = None, h
        T, H, I, E, rows = ctx.dims
        k = ctx.cfg["top_k"]
        dtype = x.dtype
        dev = x.device
        dout = dout.to(dtype).contiguous()
        need_x, need_wg = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_w = any(ctx.needs_input_grad[3:])

        dwgu = dwd = None
        if rows > 0:
            dy, dw = ops.combine_bwd(dout, y, row_src, w, k)
            dx_rows, dwgu, dwd = _ffn_backward(dy, x, ctx.wgu, ctx.wd, gu, h, offsets, kept, rows, row_src, k, need_x,
                                               need_w, hT=hT, wplan=wplan)
            if need_x:
                ones = torch.ones(T, k, dtype=torch.float32, device=dev)
                dx = ops.combine(dx_rows, row_of, ones, T, k, out_dtype=dtype)
        else:
            dw = torch.zeros(T, k, dtype=torch.float32, device=dev)
            dx = torch.zeros(T, H, dtype=dtype, device=dev) if need_x else None
            if need_w:
                dwd = torch.zeros(E, H, I, dtype=dtype, device=dev)
                dwgu = torch.zeros(E, 2 * I, H, dtype=dtype, device=dev)

        # routing rule + load-balancing loss -> router logits -> x and the gate weight
        lbw = ctx.cfg["load_balancing_weight"]
        scale_dev = (daux.detach().float() * (aux < 1.0).float()).reshape(1).contiguous()
        dz = ops.route_bwd(logits_route, idx, w, dw, ctx.cfg["temperature"], ctx.cfg["variant"], logits_aux=logits,
                           usage=usage, aux_scale=E * lbw / T, aux_scale_dev=scale_dev)
        dx_out, dwg = ops.router_bwd(dz, x, wg, base=dx if need_x else None, out=dx if need_x else None,
                                     need_dx=need_x, need_dw=need_wg)

        gate_dtype, wdtypes = ctx.param_dtypes
        grads_w = [None] * ctx.n_weights
        if need_w:
            for e in range(E):
                if ctx.needs_input_grad[3 + e]:
                    grads_w[e] = dwgu[e].to(wdtypes[e])
                if ctx.needs_input_grad[3 + E + e]:
                    grads_w[E + e] = dwd[e].to(wdtypes[E + e])
        return (dx_out if need_x else None, dwg.to(gate_dtype) if need_wg else None, None, *grads_w)


class MoDRouteFunction(Function):
    """Training branch of the reference's MoDRouter (MS/core/model.py:923-952): probabilities
    sigmoid((x . w + b) / temperature), a mask with exactly `capacity` ones at the largest of them over all
    tokens of the batch, and the straight-through weights (mask - p) + p, whose gradient goes to p unchanged.
    Returns (weights [T], probs [T], mask [T]), float32; the mask carries no gradient."""

    @staticmethod
    def forward(ctx, x, weight, bias, temperature, capacity):
        x2 = x.reshape(-1, x.shape[-1])
        w = weight if weight.dtype == x2.dtype else weight.to(x2.dtype)
        _, probs = ops.row_dot(x2, w, None if bias is None else bias.detach(), temperature, want_prob=True)
        mask, ste = ops.topk_mask_ste(probs, capacity)
        ctx.save_for_backward(x2, w, probs)
        ctx.temperature = temperature
        ctx.x_shape = x.shape
        ctx.weight_dtype = weight.dtype
        ctx.has_bias = bias is not None
        ctx.mark_non_differentiable(mask)
        return ste, probs, mask

    @staticmethod
    def backward(ctx, d_weights, d_probs, _d_mask):
        x2, w, probs = ctx.saved_tensors
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        need_b = ctx.has_bias and ctx.needs_input_grad[2]
        gw = None if d_weights is None else d_weights.float()
        gp = None if d_probs is None else d_probs.float()
        gl, db = ops.mod_route_bwd(probs, gw, gp, ctx.temperature, need_bias=need_b)
        dx, dw = ops.router_bwd(gl.view(-1, 1), x2, w.reshape(1, -1), need_dx=need_x, need_dw=need_w)
        return (dx.view(ctx.x_shape) if need_x else None,
                dw.to(ctx.weight_dtype) if need_w else None,
                db if need_b else None, None, None)


def moe_variant(routing: str) -> int:
    return {"softmax_topk": ROUTE_SOFTMAX_TOPK, "topk_softmax": ROUTE_TOPK_SOFTMAX}[routing]
