"""CPU oracle for the sparse-layer path (RMSNorm, RoPE/GQA, MoE routing, capacity
dispatch, SwiGLU experts, combine, aux loss, MoD selection).

THIS FILE IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only the tests, the smoke
check and the CPU-baseline leg of the benchmark may import it.  The product
package never imports it and has no CPU fallback.

Every function restates, in plain torch-on-CPU (float32 unless stated), one
function of the reference's own PyTorch path and cites the lines it follows
(paths relative to the reference checkout; MS = Src/Main_Scripts).  Loops that
the reference writes as Python loops are kept as literal loops (``*_loop``)
and additionally given a vectorised twin; tests check the twins against each
other, against closed forms and against brute force.

Pinning status (what independent check fixes each function) is listed in
``PINNING`` below; a function with no independent check would be marked
"parity unpinned" there.  The reference's own tests hold no golden vectors
for this path (they assert shapes and finiteness only), so no function is
pinned by a reference fixture.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

PINNING = {
    "rmsnorm": "closed form in float64 numpy; unit row-RMS invariant; torch.nn.functional.rms_norm",
    "rope_table": "closed form with math.cos/math.sin in float64; pos 0 and d 0 special cases",
    "rope_apply": "2x2 rotation closed form per pair in float64; norm preservation; R(p)R(-p)=I; relative-position identity",
    "fused_rope_table": "both halves (cos and sin) against math.cos/math.sin of pos * theta^(-d/half) in float64; "
                        "sin(1) > 0 at position 1; agreement with both halves of rope_table",
    "fused_rope_apply": "per-element 2x2 rotation in float64 with an offset; equals rope_apply with a half-width table",
    "router_logits": "float64 matmul",
    "route_softmax_topk_renorm": "brute-force full sort on tiny inputs; index set equals route_topk_softmax; weights sum to 1",
    "route_topk_softmax": "brute-force full sort on tiny inputs; weights sum to 1",
    "capacity": "python expression is the specification; table of known values incl. a truncation case",
    "dispatch_loop": "literal restatement; stable-counting-sort closed form (dispatch_vectorized); C restatement; invariants",
    "combine_loop": "literal restatement; equals no-capacity formulation when nothing is dropped; linearity in weights",
    "swiglu_expert": "float64 closed form with explicit sigmoid",
    "moe_forward_nocap": "dense brute force: sum over all experts of mask*weight*expert(x)",
    "aux_loss": "uniform routing gives exactly load_balancing_weight; float64 closed form",
    "mod_router_probs": "float64 closed form 1/(1+exp(-(x.w+b)/T)) with bias != 0 and temperature != 1; "
                        "w = 0 gives sigmoid(b/T); p(x)+p(-x) = 1 without bias",
    "mod_router_eval_mask": "sorted-threshold brute force",
    "mod_router_train": "mask = brute-force ranking (exactly int(N*cf) ones, at the largest probabilities); the weights' value "
                        "is the mask to one ulp; d weights / d logit = p(1-p)/T against the float64 closed form, with a "
                        "non-constant cotangent; aux = (k/N - cf)^2 closed form and no gradient",
    "mod_select_per_sequence": "argsort brute force (composition defined by the benchmark config, not a reference function)",
    "mod_moe_block": "scores against a float64 matmul + bias; selection against a brute-force sort; skipped tokens "
                     "bit-identical to the input, kept tokens = input + capacity layer output",
    "dispatch_plan_vectorized": "same three-formulation check as dispatch_loop (slot, hist, kept)",
    "dispatch_vectorized": "equals dispatch_loop element for element",
    "combine_vectorized": "equals combine_loop",
    "experts_on_slots": "per-slot swiglu_expert (itself pinned in float64); empty slots stay zero",
    "moe_nocap_compute": "dense brute force over all experts",
    "moe_forward_capacity": "composition of pinned parts; equals the no-capacity layer when nothing is dropped; "
                            "hand-worked drop cases",
    "rmsnorm_backward": "torch.autograd of rmsnorm in float64; torch.autograd.gradcheck",
    "rope_backward": "torch.autograd of rope_apply; R(p)^T = R(-p)",
    "swiglu_backward": "torch.autograd of gate*silu(up) in float64; gradcheck",
    "fused_loss": "float64 logsumexp closed form; uniform logits give log(V); torch.autograd for the gradient",
    "clip_grad_norm": "closed form sqrt(sum of squares) and scaling by max_norm/(norm+1e-6)",
    "attention_standard": "float64 brute force per query (explicit loop over allowed keys); F.scaled_dot_product_attention(is_causal=True); "
                          "4-D masks and the explicit dropout mask against a float64 sum written out per element",
    "attention_dropout_keep": "published values of MurmurHash3's fmix32 (0, 1, 2) on both sides of their thresholds; keep rate within "
                              "4 sigma; zero correlation between seeds, heads, batch entries and neighbouring elements",
    "gqa_forward": "composition of pinned parts; equals per-head attention with repeat_interleave done by hand",
    "layer_grads": "is torch.autograd over the forward restatements above (what the reference itself trains with); "
                   "gradcheck in float64 on the no-capacity layer with fixed routing",
}


# --------------------------------------------------------------------------- RMSNorm
def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float = 1e-6) -> torch.Tensor:
    """MS/core/model.py:263-299 (RMSNorm._norm_pytorch + forward fallback).

    float32 math on the up-cast input, weight applied in float32, result cast
    back to the input dtype.
    """
    in_dtype = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(-1, keepdim=True)
    y = xf * torch.rsqrt(var + eps)
    if weight is not None:
        y = y * weight.float()
    return y.to(in_dtype)


# --------------------------------------------------------------------------- RoPE
def rope_table(seq_len: int, dim: int, theta: float = 10000.0,
               scaling_factor: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """MS/core/model.py:378-402 (RotaryEmbedding._build_pytorch_cache).

    inv_freq in float64, positions in float32, outer product promoted to
    float64, cos/sin evaluated in float64 and stored as float32 [L, dim] with
    the two halves duplicated.
    """
    inv_freq = 1.0 / (theta ** (torch.arange(0, dim, 2, dtype=torch.float64) / dim))
    t = torch.arange(seq_len, dtype=torch.float32)
    if scaling_factor is not None:
        t = t / scaling_factor
    freqs = torch.outer(t, inv_freq)          # float32 x float64 -> float64
    emb = torch.cat((freqs, freqs), dim=-1).double()
    return emb.cos().float(), emb.sin().float()


def fused_rope_table(max_seq_len: int, head_dim: int, theta: float = 10000.0):
    """MS/core/cuda_opt_wrapper.py:350-363 (FusedRoPE._precompute_pytorch_cache).

    Half-width table [max_seq, head_dim/2] evaluated entirely in float32.
    """
    half = head_dim // 2
    freqs = 1.0 / (theta ** (torch.arange(0, half, dtype=torch.float32) / half))
    pos = torch.arange(max_seq_len, dtype=torch.float32)
    ang = pos.unsqueeze(1) * freqs.unsqueeze(0)
    return torch.cos(ang), torch.sin(ang)


def rope_apply(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor):
    """MS/core/model.py:470-524 (apply_rotary_pos_emb_optimized).

    q [B,Hq,L,D], k [B,Hkv,L,D]; cos/sin [L, D] (only the first D/2 columns are
    used).  Rotate-half convention.  A bf16 input times the float32 table
    promotes to float32; the policy of this build is to round that float32
    result once to the input dtype, which is what ``.to(q.dtype)`` does here.
    """
    def rot(x):
        x1, x2 = x.float().chunk(2, dim=-1)
        half = x1.shape[-1]
        c = cos[..., :half].float().unsqueeze(0).unsqueeze(0)
        s = sin[..., :half].float().unsqueeze(0).unsqueeze(0)
        return torch.cat([x1 * c - x2 * s, x1 * s + x2 * c], dim=-1).to(x.dtype)
    return rot(q), rot(k)


def fused_rope_apply(q, k, cos_half, sin_half, position_offset: int = 0):
    """MS/core/cuda_opt_wrapper.py:391-425 (FusedRoPE._pytorch_fallback)."""
    L = q.shape[2]
    pos = torch.arange(position_offset, position_offset + L)
    return rope_apply(q, k, cos_half[pos], sin_half[pos])


# --------------------------------------------------------------------------- router + routing
def router_logits(x: torch.Tensor, gate_weight: torch.Tensor) -> torch.Tensor:
    """MS/core/model.py:1124,1169 (self.gate = nn.Linear(H, E, bias=False)).

    float32 logits from float32 accumulation of the (possibly bf16) operands.
    """
    return F.linear(x.float(), gate_weight.float())


def route_softmax_topk_renorm(logits: torch.Tensor, k: int, temperature: float = 1.0):
    """MS/core/model.py:1200-1217 (MoEFFNLayer._pytorch_routing, eval mode: no noise)."""
    scaled = logits / temperature
    probs = F.softmax(scaled, dim=-1)
    top_p, top_i = torch.topk(probs, k, dim=-1)
    top_p = top_p / (top_p.sum(dim=-1, keepdim=True) + 1e-9)
    return top_i, top_p


def route_topk_softmax(logits: torch.Tensor, k: int, temperature: float = 1.0):
    """MS/core/moe_cuda_wrapper.py:229-233 (MoECUDAOps.topk_gating, PyTorch branch)."""
    scaled = logits / temperature
    top_v, top_i = torch.topk(scaled, k, dim=-1)
    return top_i, F.softmax(top_v, dim=-1)


def capacity(total_tokens: int, top_k: int, num_experts: int, capacity_factor: float) -> int:
    """MS/core/moe_cuda_wrapper.py:440 (also MS/cuda_debug_script.py:220)."""
    return int((total_tokens * top_k / num_experts) * capacity_factor)


# --------------------------------------------------------------------------- dispatch
def dispatch_loop(tokens: torch.Tensor, top_k_indices: torch.Tensor, num_experts: int, cap: int):
    """MS/core/moe_cuda_wrapper.py:295-326 (MoECUDAOps._pytorch_dispatch), literal loop.

    First come first served in (token, choice) order; an assignment whose
    expert is already full is dropped.
    """
    T, H = tokens.shape
    k = top_k_indices.shape[1]
    expert_inputs = torch.zeros(num_experts, cap, H, dtype=tokens.dtype)
    token_map = torch.full((num_experts, cap), -1, dtype=torch.int32)
    positions = [0] * num_experts
    idx = top_k_indices.tolist()
    for t in range(T):
        for j in range(k):
            e = idx[t][j]
            pos = positions[e]
            if pos < cap:
                expert_inputs[e, pos] = tokens[t]
                token_map[e, pos] = t * k + j
                positions[e] += 1
    return expert_inputs, token_map


def dispatch_plan_vectorized(top_k_indices: torch.Tensor, num_experts: int, cap: int):
    """Closed form of the loop above on the integer side: a stable counting sort.

    Returns (token_map [E,C] int32, slot [T*k] int32 (-1 = dropped),
    hist [E] int64 (pre-capacity), kept [E] int64).
    """
    flat = top_k_indices.reshape(-1).to(torch.int64).numpy()
    n = flat.shape[0]
    order = np.argsort(flat, kind="stable")
    hist = np.bincount(flat, minlength=num_experts).astype(np.int64)
    starts = np.concatenate([[0], np.cumsum(hist)[:-1]])
    rank = np.empty(n, dtype=np.int64)
    rank[order] = np.arange(n) - np.repeat(starts, hist)
    slot = np.where(rank < cap, rank, -1).astype(np.int32)
    token_map = np.full((num_experts, cap), -1, dtype=np.int32)
    keep = slot >= 0
    token_map[flat[keep], slot[keep]] = np.nonzero(keep)[0].astype(np.int32)
    kept = np.minimum(hist, cap)
    return (torch.from_numpy(token_map), torch.from_numpy(slot),
            torch.from_numpy(hist), torch.from_numpy(kept))


def dispatch_vectorized(tokens, top_k_indices, num_experts: int, cap: int):
    token_map, _, _, _ = dispatch_plan_vectorized(top_k_indices, num_experts, cap)
    k = top_k_indices.shape[1]
    H = tokens.shape[1]
    expert_inputs = torch.zeros(num_experts, cap, H, dtype=tokens.dtype)
    occ = token_map >= 0
    expert_inputs[occ] = tokens[(token_map[occ] // k).long()]
    return expert_inputs, token_map


# --------------------------------------------------------------------------- experts
def swiglu_expert(x: torch.Tensor, gate_up_weight: torch.Tensor, down_weight: torch.Tensor,
                  intermediate_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """MS/core/model.py:1071-1088 (SwiGLUExpert.forward).

    gate = first I output rows of the fused [2I,H] weight, up = last I rows;
    y = down(silu(gate) * up).  ``intermediate_dtype`` optionally rounds the
    [n, I] intermediate once (bf16 path policy of this build).
    """
    gu = F.linear(x.float(), gate_up_weight.float())
    g, u = gu.chunk(2, dim=-1)
    h = F.silu(g) * u
    if intermediate_dtype is not None:
        h = h.to(intermediate_dtype).float()
    return F.linear(h, down_weight.float())


def experts_on_slots(expert_inputs, token_map, gate_up_weights, down_weights,
                     intermediate_dtype=None):
    """MS/core/moe_cuda_wrapper.py:452-457 (per-expert loop over occupied slots)."""
    out = torch.zeros(expert_inputs.shape, dtype=torch.float32)
    for e in range(expert_inputs.shape[0]):
        mask = token_map[e] >= 0
        if mask.any():
            out[e][mask] = swiglu_expert(expert_inputs[e][mask], gate_up_weights[e],
                                         down_weights[e], intermediate_dtype)
    return out


# --------------------------------------------------------------------------- combine
def combine_loop(expert_outputs, token_map, top_k_weights, num_tokens: int, k: int):
    """MS/core/moe_cuda_wrapper.py:328-359 (MoECUDAOps._pytorch_combine), literal loop.

    Ascending expert id, then ascending slot; weights are not renormalised
    after drops.
    """
    E, C, H = expert_outputs.shape
    out = torch.zeros(num_tokens, H, dtype=expert_outputs.dtype)
    tm = token_map.tolist()
    for e in range(E):
        for pos in range(C):
            m = tm[e][pos]
            if m < 0:
                continue
            t, j = m // k, m % k
            if t >= num_tokens:
                continue
            out[t] += top_k_weights[t, j] * expert_outputs[e, pos]
    return out


def combine_vectorized(expert_outputs, token_map, top_k_weights, num_tokens: int, k: int):
    """Same sums in the same order: one index_add_ per expert (slots of one
    expert belong to distinct tokens, so each token gets one add per expert)."""
    E, C, H = expert_outputs.shape
    out = torch.zeros(num_tokens, H, dtype=expert_outputs.dtype)
    w_flat = top_k_weights.reshape(-1)
    for e in range(E):
        occ = token_map[e] >= 0
        m = token_map[e][occ].long()
        if m.numel() == 0:
            continue
        out.index_add_(0, m // k, w_flat[m].unsqueeze(-1).to(expert_outputs.dtype) * expert_outputs[e][occ])
    return out


# --------------------------------------------------------------------------- no-capacity MoE
def moe_nocap_compute(x, indices, probs, gate_up_weights, down_weights, intermediate_dtype=None):
    """MS/core/model.py:1219-1242 (MoEFFNLayer._compute_experts_vectorized)."""
    out = torch.zeros(x.shape, dtype=torch.float32)
    xf = x.float()
    for e in range(len(gate_up_weights)):
        mask = indices == e
        tok = mask.any(dim=-1).nonzero(as_tuple=True)[0]
        if tok.numel() == 0:
            continue
        w = probs[mask].view(-1)
        y = swiglu_expert(xf[tok], gate_up_weights[e], down_weights[e], intermediate_dtype)
        out.index_add_(0, tok, y * w.unsqueeze(-1))
    return out


# --------------------------------------------------------------------------- aux loss
def aux_loss(gate_logits: torch.Tensor, top_k_indices: torch.Tensor, num_experts: int,
             load_balancing_weight: float = 0.01) -> torch.Tensor:
    """MS/core/model.py:1190-1192,1244-1263 (softmax of the un-tempered logits, mean
    over tokens, times the pre-capacity usage histogram)."""
    T, k = top_k_indices.shape
    gate_probs = F.softmax(gate_logits.float(), dim=-1)
    usage = torch.zeros(num_experts)
    for j in range(k):
        usage += torch.bincount(top_k_indices[:, j].long(), minlength=num_experts).float()
    usage = usage / (T * k + 1e-9)
    importance = gate_probs.mean(dim=0)
    return torch.clamp(torch.sum(usage * importance) * num_experts * load_balancing_weight, max=1.0)


# --------------------------------------------------------------------------- whole layers
def moe_forward_capacity(x, gate_weight, gate_up_weights, down_weights, k: int,
                         capacity_factor: float = 1.25, temperature: float = 1.0,
                         routing: str = "softmax_topk", load_balancing_weight: float = 0.01,
                         logit_bias: Optional[torch.Tensor] = None,
                         logits_override: Optional[torch.Tensor] = None,
                         intermediate_dtype=None, literal_loops: bool = False):
    """MS/core/moe_cuda_wrapper.py:413-478 (capacity MoEFFNLayer.forward, eval mode) with
    the routing rule selectable: ``softmax_topk`` = MS/core/model.py:1200-1217,
    ``topk_softmax`` = MS/core/moe_cuda_wrapper.py:229-233.

    x is [B, L, H] or [T, H].  Returns a dict with every intermediate that the
    parity tests compare.  ``logit_bias`` is the benchmark's per-expert skew;
    ``logits_override`` replaces the router output so that two implementations
    can be compared on bit-equal logits.
    """
    shape = x.shape
    xf = x.reshape(-1, shape[-1])
    T = xf.shape[0]
    E = gate_weight.shape[0]
    logits = router_logits(xf, gate_weight) if logits_override is None else logits_override.float()
    if logit_bias is not None and logits_override is None:
        logits = logits + logit_bias.float()
    if routing == "softmax_topk":
        idx, w = route_softmax_topk_renorm(logits, k, temperature)
    elif routing == "topk_softmax":
        idx, w = route_topk_softmax(logits, k, temperature)
    else:
        raise ValueError(routing)
    C = capacity(T, k, E, capacity_factor)
    disp = dispatch_loop if literal_loops else dispatch_vectorized
    comb = combine_loop if literal_loops else combine_vectorized
    expert_inputs, token_map = disp(xf.float(), idx, E, C)
    expert_outputs = experts_on_slots(expert_inputs, token_map, gate_up_weights, down_weights,
                                      intermediate_dtype)
    out = comb(expert_outputs, token_map, w, T, k)
    aux = aux_loss(logits, idx, E, load_balancing_weight)
    _, slot, hist, kept = dispatch_plan_vectorized(idx, E, C)
    return {
        "out": out.reshape(shape), "aux": aux, "logits": logits, "indices": idx, "weights": w,
        "capacity": C, "token_map": token_map, "slot": slot, "hist": hist, "kept": kept,
        "expert_outputs": expert_outputs,
    }


def moe_forward_nocap(x, gate_weight, gate_up_weights, down_weights, k: int,
                      temperature: float = 1.0, load_balancing_weight: float = 0.01,
                      logits_override=None, intermediate_dtype=None):
    """MS/core/model.py:1160-1198 (MoEFFNLayer.forward, eval mode, PyTorch routing)."""
    shape = x.shape
    xf = x.reshape(-1, shape[-1])
    E = gate_weight.shape[0]
    logits = router_logits(xf, gate_weight) if logits_override is None else logits_override.float()
    idx, w = route_softmax_topk_renorm(logits, k, temperature)
    out = moe_nocap_compute(xf, idx, w, gate_up_weights, down_weights, intermediate_dtype)
    return {"out": out.reshape(shape), "aux": aux_loss(logits, idx, E, load_balancing_weight),
            "logits": logits, "indices": idx, "weights": w}


# --------------------------------------------------------------------------- MoD
def mod_router_probs(x, router_weight, router_bias, temperature: float = 1.0):
    """MS/core/model.py:926-936 (MoDRouter.forward: Linear(H,1) / temperature -> sigmoid)."""
    logit = F.linear(x.float(), router_weight.float(),
                     None if router_bias is None else router_bias.float())
    return torch.sigmoid(logit / temperature)


def mod_router_eval_mask(probs: torch.Tensor, capacity_factor: float):
    """MS/core/model.py:938-940,984-995 (inference branch: k-th value threshold).

    capacity counts over ALL tokens of the batch; tokens with prob >= the
    max(1, N - capacity)-th smallest value are kept, which keeps capacity+1
    tokens when there are no ties.
    """
    n = probs.numel()
    cap = int(n * capacity_factor)
    thr = probs.flatten().kthvalue(max(1, n - cap))[0]
    return (probs >= thr).float()


def mod_router_train(x, router_weight, router_bias, temperature: float = 1.0, capacity_factor: float = 0.5):
    """MS/core/model.py:923-965 (MoDRouter.forward, training branch, up to where its placeholder code begins).

    -> (routing_weights [B,L,1] = mask - p.detach() + p, routing_probs [B,L,1], mask [B,L,1], aux_loss).
    The mask has exactly min(int(B*L*cf), B*L) ones, at the largest probabilities over the whole batch
    (torch.topk; among equal probabilities the library picks).  aux = mse(mask.mean(), cf)."""
    B, L, _ = x.shape
    probs = mod_router_probs(x, router_weight, router_bias, temperature)     # [B, L, 1]
    total = B * L
    cap = int(total * capacity_factor)
    flat = probs.view(-1)
    _, top = torch.topk(flat, k=min(cap, total))
    mask = torch.zeros_like(flat)
    mask[top] = 1.0
    mask = mask.view(B, L, 1).detach()
    weights = mask - probs.detach() + probs
    aux = F.mse_loss(mask.mean(), torch.tensor(capacity_factor))
    return weights, probs, mask, aux


def mod_select_per_sequence(scores: torch.Tensor, keep: int) -> torch.Tensor:
    """Benchmark-defined composition (not a reference function): per sequence keep
    the ``keep`` highest scores; return their positions in ascending order,
    shape [B, keep] int64.  Ties are broken toward the lower position."""
    B, L = scores.shape
    # stable descending sort = ascending sort of the negated scores with stable order
    order = torch.sort(-scores.float(), dim=-1, stable=True)[1][:, :keep]
    return torch.sort(order, dim=-1)[0]


def mod_moe_block(x, mod_weight, mod_bias, keep, moe_kwargs):
    """Composition used by the fine-grained benchmark config: score every token,
    keep the top ``keep`` per sequence, run the capacity MoE on the gathered
    tokens (batch-major, ascending position), add the result onto the residual
    stream at the kept positions; skipped tokens pass through unchanged."""
    B, L, H = x.shape
    scores = F.linear(x.float(), mod_weight.float(),
                      None if mod_bias is None else mod_bias.float()).squeeze(-1)
    sel = mod_select_per_sequence(scores, keep)                      # [B, keep]
    rows = (sel + torch.arange(B).unsqueeze(1) * L).reshape(-1)      # flat token ids
    gathered = x.reshape(-1, H)[rows]
    res = moe_forward_capacity(gathered, **moe_kwargs)
    out = x.reshape(-1, H).float().clone()
    out[rows] += res["out"].reshape(-1, H)
    res.update({"block_out": out.reshape(B, L, H), "selected": sel, "scores": scores})
    return res


# --------------------------------------------------------------------------- backward pass
def rmsnorm_backward(x: torch.Tensor, weight: Optional[torch.Tensor], dy: torch.Tensor, eps: float = 1e-6):
    """MS/core/cuda_opt_wrapper.py:119-142 (RMSNormFunction.backward), float32 math.
    Returns (dx in x's dtype, dw float32 or None)."""
    xf, gf = x.float().reshape(-1, x.shape[-1]), dy.float().reshape(-1, x.shape[-1])
    hidden = xf.shape[-1]
    rstd = torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    dw = (gf * xf * rstd).sum(0) if weight is not None else None
    g = gf * weight.float().unsqueeze(0) if weight is not None else gf
    gi = g * rstd
    mean_grad = (gi * xf).sum(-1, keepdim=True) / hidden
    dx = gi - xf * mean_grad * rstd.pow(2)
    return dx.reshape(x.shape).to(x.dtype), dw


def rope_backward(dq: torch.Tensor, dk: torch.Tensor, cos_half: torch.Tensor, sin_half: torch.Tensor,
                  position_offset: int = 0):
    """MS/core/cuda_opt_wrapper.py:180-207 (RoPEFunction.backward): inverse rotation."""
    L = dq.shape[2]
    pos = torch.arange(position_offset, position_offset + L)
    def inv(g):
        half = g.shape[-1] // 2
        c = cos_half[pos][..., :half].float().unsqueeze(0).unsqueeze(0)
        s = sin_half[pos][..., :half].float().unsqueeze(0).unsqueeze(0)
        g1, g2 = g.float()[..., :half], g.float()[..., half:]
        return torch.cat([g1 * c + g2 * s, -g1 * s + g2 * c], dim=-1).to(g.dtype)
    return inv(dq), inv(dk)


def swiglu_backward(gate: torch.Tensor, up: torch.Tensor, dout: torch.Tensor):
    """MS/core/cuda_opt_wrapper.py:237-254 (SwiGLUFunction.backward; out = gate * silu(up))."""
    g, u, d = gate.float(), up.float(), dout.float()
    sig = torch.sigmoid(u)
    dgate = d * (u * sig)
    dup = d * g * (sig + u * sig * (1 - sig))
    return dgate.to(gate.dtype), dup.to(up.dtype)


def layer_grads(forward, tensors, cotangents):
    """Gradients the reference obtains from PyTorch autograd (it trains the MoE layer through
    MS/core/model.py with plain autograd): differentiates ``forward(*leaves)`` -- a callable built
    from the forward restatements above that returns a tuple of tensors -- against ``cotangents``.
    All leaves are float32 copies with requires_grad; returns the list of their gradients."""
    leaves = [t.detach().float().clone().requires_grad_() for t in tensors]
    outs = forward(*leaves)
    if isinstance(outs, torch.Tensor):
        outs = (outs,)
    loss = sum((o.float() * c.float()).sum() for o, c in zip(outs, cotangents))
    return list(torch.autograd.grad(loss, leaves, allow_unused=True))


# --------------------------------------------------------------------------- training-step ops
def fused_loss(logits: torch.Tensor, labels: torch.Tensor, loss_weights: Optional[torch.Tensor] = None,
               pad_token_id: int = -100):
    """MS/training/cuda_kernels.py:191-249 (FusedLoss._pytorch_fallback), float32 math, with the
    validity rule of the fused kernel (MS/training/fused_loss.cu:83-84: a label equal to the pad id or
    outside [0, V) is ignored).  Returns the dict of the reference; ``loss`` is differentiable."""
    V = logits.shape[-1]
    lg = logits.reshape(-1, V).float()
    lb = labels.reshape(-1).long()
    mask = ((lb != pad_token_id) & (lb >= 0) & (lb < V)).float()
    n_valid = mask.sum()
    safe = torch.where(mask.bool(), lb, torch.zeros_like(lb))
    per_tok = F.cross_entropy(lg, safe, reduction="none")
    per_tok = torch.where(torch.isfinite(per_tok), per_tok, torch.full_like(per_tok, 10.0))
    acc = ((lg.argmax(-1) == lb).float() * mask).sum() / n_valid.clamp(min=1.0)
    raw = (per_tok * mask).sum() / n_valid.clamp(min=1.0)
    if loss_weights is not None:
        w = loss_weights.reshape(-1).float()
        loss = (per_tok * w * mask).sum() / (w * mask).sum().clamp(min=1e-8)
    else:
        loss = (per_tok * mask).sum() / n_valid.clamp(min=1e-8)
    ppl = torch.exp(torch.clamp(raw.detach(), min=0.0, max=15.0)) if n_valid > 0 else torch.tensor(float("inf"))
    return {"loss": loss, "raw_loss": raw.detach(), "perplexity": ppl, "valid_tokens": n_valid, "accuracy": acc}


def clip_grad_norm(grads, max_norm: float):
    """MS/training/cuda_kernels.py:340-342 (torch.nn.utils.clip_grad_norm_) restated on a list of
    gradient tensors: returns (total L2 norm float32, list of clipped copies)."""
    total = torch.sqrt(sum((g.float() ** 2).sum() for g in grads)) if grads else torch.tensor(0.0)
    coef = max_norm / (total + 1e-6)
    out = [(g.float() * coef).to(g.dtype) if coef < 1.0 else g.clone() for g in grads]
    return total, out


# --------------------------------------------------------------------------- attention
def attention_standard(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                       attention_mask=None, dropout_keep=None, dropout_p: float = 0.0) -> torch.Tensor:
    """MS/core/model.py:757-838 (GroupedQueryAttention._standard_attention).
    q [B,H,L,D], k/v [B,H,Lk,D] (already expanded to H heads), Lk >= L.  Scores and softmax in float32,
    causal positions filled with -1e4, probabilities cast to the input dtype before the second matmul,
    output [B, L, H*D] in the input dtype.
    With cached keys in front (Lk > L, model.py:700-704) query i sits at position i + Lk - L.  The
    reference's own [L, L] mask only broadcasts against [L, Lk] scores for L = 1 (one new token, which
    then sees every key); the diagonal used here is that case's generalisation, and equals what slicing
    the last L query rows out of a full-length call gives.
    attention_mask (1 = attend, 0 = masked) adds (1 - mask) * -1e4 to the scores after the causal fill
    (model.py:819-824): [B, Lk] for every query and head (unsqueezed as there), or 4-D [B, 1, L, Lk] as given.
    dropout_keep [B,H,L,Lk] bool with dropout_p: nn.Dropout on the weights (model.py:831-833) with the mask
    made explicit: kept weights are scaled by 1 / (1 - p), the others are zero."""
    B, H, L, D = q.shape
    Lk = k.shape[2]
    scores = torch.matmul(q.float(), k.float().transpose(-2, -1)) * scale
    causal = torch.triu(torch.ones(L, Lk, dtype=torch.bool), diagonal=1 + Lk - L)
    scores = scores.masked_fill(causal, -1e4)
    if attention_mask is not None:
        m = attention_mask.float()
        if m.dim() == 2:
            m = m[:, None, None, :]
        scores = scores + (1.0 - m) * -1e4
    scores = scores - scores.detach().amax(dim=-1, keepdim=True)
    w = F.softmax(scores, dim=-1, dtype=torch.float32).to(q.dtype)
    if dropout_keep is not None:
        w = (w.float() * dropout_keep.to(torch.float32) / (1.0 - dropout_p)).to(q.dtype)
    out = torch.matmul(w.float(), v.float()).to(q.dtype)
    return out.transpose(1, 2).reshape(B, L, H * D)


def attention_dropout_keep(seed: int, B: int, H: int, L: int, Lk: int, dropout_p: float) -> torch.Tensor:
    """The keep / drop decision of the HIP attention kernels' dropout as a bool tensor [B, H, L, Lk].  No
    counterpart in the reference (nn.Dropout draws from torch's generator, which a tiled kernel cannot
    replay): element (b, h, i, j) is kept iff fmix32((i * Lk + j) ^ head_key(seed, b * H + h)) >= p * 2^32,
    fmix32 the finaliser of MurmurHash3 (csrc/attention_extra.hpp states the same function for the device)."""
    M = 0xFFFFFFFF
    seed &= 0xFFFFFFFFFFFFFFFF
    lo, hi = seed & M, seed >> 32
    bh = np.arange(B * H, dtype=np.uint64)
    x = (np.uint64(lo) ^ ((bh * np.uint64(0x9E3779B1)) & np.uint64(M))) & np.uint64(M)
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x2C1B3C6D)) & np.uint64(M)
    x ^= np.uint64(hi)
    x ^= x >> np.uint64(12)
    y = (np.arange(L * Lk, dtype=np.uint64)[None, :] & np.uint64(M)) ^ x[:, None]
    y ^= y >> np.uint64(16)
    y = (y * np.uint64(0x85EBCA6B)) & np.uint64(M)
    y ^= y >> np.uint64(13)
    y = (y * np.uint64(0xC2B2AE35)) & np.uint64(M)
    y ^= y >> np.uint64(16)
    t = dropout_p * 4294967296.0
    threshold = M if t >= 4294967295.0 else int(t)
    return torch.from_numpy((y >= np.uint64(threshold)).reshape(B, H, L, Lk))


def gqa_forward(x: torch.Tensor, wq: torch.Tensor, wk: torch.Tensor, wv: torch.Tensor, wo: torch.Tensor,
                num_heads: int, num_kv_heads: int, theta: float = 10000.0, past_key_value=None,
                use_cache: bool = False, attention_mask=None):
    """MS/core/model.py:663-731 (GroupedQueryAttention.forward): projections (float32 accumulation,
    rounded to the input dtype like nn.Linear), RoPE at positions 0..L-1 (also with a cache, 690-698),
    cached keys/values concatenated in front (700-704), KV heads repeated, attention, o_proj.
    Returns the output, and the (k, v) cache as well when use_cache is set (706-708, 729-731)."""
    B, L, H = x.shape
    D = wq.shape[0] // num_heads
    lin = lambda a, w: F.linear(a.float(), w.float()).to(a.dtype)
    q = lin(x, wq).view(B, L, num_heads, D).transpose(1, 2)
    k = lin(x, wk).view(B, L, num_kv_heads, D).transpose(1, 2)
    v = lin(x, wv).view(B, L, num_kv_heads, D).transpose(1, 2)
    cos, sin = rope_table(L, D, theta)
    q, k = rope_apply(q, k, cos, sin)
    if past_key_value is not None:
        k = torch.cat([past_key_value[0], k], dim=2)
        v = torch.cat([past_key_value[1], v], dim=2)
    cache = (k, v)
    rep = num_heads // num_kv_heads
    if rep > 1:
        k = k.repeat_interleave(rep, dim=1)
        v = v.repeat_interleave(rep, dim=1)
    a = attention_standard(q, k, v, D ** -0.5, attention_mask)
    out = lin(a, wo)
    return (out, cache) if use_cache else out
