"""The benchmark configurations at their full sizes on the GPU.  Each test checks (a) every integer
artefact bit for bit, (b) EVERY output row of the float pipeline against the oracle's whole capacity
layer (fed the GPU's logits so that routing is compared on bit-equal inputs; the logits themselves are
compared with the oracle's own router product, and the tokens that route differently on those are counted
and must be near-ties; the oracle runs the 16384-token prefill layer in seconds on the host cores), and (c) size-independent properties:
dispatch -> combine round trip, conservation of assignments, untouched skip tokens."""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import sparse_layer_oracle as O

pytestmark = pytest.mark.gpu
BF16_TOL = 2e-2


def rel_err(got, ref):
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    return (got - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)


def _check_routing_and_plan(p, w, T):
    logits = p["logits"].cpu()
    ri, rw = O.route_softmax_topk_renorm(logits, w.top_k, 1.0)
    assert torch.equal(p["indices"].cpu().long(), ri)
    assert (p["weights"].cpu() - rw).abs().max().item() <= 1e-5
    C = O.capacity(T, w.top_k, w.num_experts, w.capacity_factor)
    assert p["capacity"] == C
    tm, slot, hist, kept, dropped = c_oracle.fcfs_dispatch(ri.numpy(), w.num_experts, C)
    assert np.array_equal(p["token_map"].cpu().numpy(), tm)
    assert np.array_equal(p["slot"].cpu().numpy(), slot)
    assert np.array_equal(p["hist"].cpu().numpy(), hist) and np.array_equal(p["kept"].cpu().numpy(), kept)
    assert int(kept.sum()) + dropped == T * w.top_k
    assert abs(p["aux"].item() - O.aux_loss(logits, ri, w.num_experts, 0.01).item()) <= 1e-6
    return ri, rw, tm, kept, dropped


def _check_logits_against_own_router(p, w, x_flat, T):
    """The GPU's logits against the oracle's OWN router product on the same inputs (MS/core/model.py:1124,1169),
    so that a router kernel computing wrong but self-consistent logits cannot pass; then the number of tokens
    the oracle routes differently on its own logits.  Such a token must be a near-tie: the gap between its
    k-th and (k+1)-th own logit is within the float32 bar of the logits, anything else is a routing error."""
    own = O.router_logits(x_flat.cpu(), w.gate.cpu())
    if w.logit_bias is not None:
        own = own + w.logit_bias.cpu()
    got = p["logits"].cpu()
    assert got.shape == own.shape == (T, w.num_experts)
    err = rel_err(got, own)
    own_idx = O.route_softmax_topk_renorm(own, w.top_k, 1.0)[0]
    differs = (own_idx != p["indices"].cpu().long()).any(-1)
    mism = int(differs.sum())
    srt = torch.sort(own, dim=-1, descending=True)[0][:, : w.top_k + 1]
    gap = (srt[:, :-1] - srt[:, 1:]).amin(-1)
    bar = 2e-5 * own.abs().max().item()     # a flip needs a gap within twice the logits' 1e-5 bar
    worst = gap[differs].max().item() if mism else 0.0
    print(f"{w.name}: logits vs the oracle's own router rel err {err:.2e}; tokens routed differently on the "
          f"oracle's own logits: {mism} of {T} (largest logit gap among them {worst:.2e}, bar {bar:.2e})", flush=True)
    assert err <= 1e-5
    assert mism <= max(1, T // 500) and worst <= bar
    return mism


def _check_sampled_outputs(out, x_flat, w, ri, rw, tm, kept, tokens_to_check, k):
    """Recomputes the layer output for a few tokens on the CPU (all their kept choices, ascending
    expert order) and compares with the GPU output rows."""
    slot_of = {}
    for e in range(w.num_experts):
        for pos in range(int(kept[e])):
            slot_of[int(tm[e, pos])] = e
    per_expert = {}
    for t in tokens_to_check:
        for j in range(k):
            a = t * k + j
            if a in slot_of:
                per_expert.setdefault(slot_of[a], []).append((t, j))
    ref = {t: torch.zeros(w.hidden) for t in tokens_to_check}
    for e in sorted(per_expert):
        toks = [t for t, _ in per_expert[e]]
        y = O.swiglu_expert(x_flat[toks].float().cpu(), w.gate_up[e].float().cpu(), w.down[e].float().cpu())
        for (t, j), row in zip(per_expert[e], y):
            ref[t] += rw[t, j] * row
    got = out.reshape(-1, w.hidden)[tokens_to_check].float().cpu()
    want = torch.stack([ref[t] for t in tokens_to_check])
    return rel_err(got, want)


def _oracle_layer(w, x_cpu, p):
    """The oracle's capacity layer on the same inputs and weights, routed by the GPU's logits, with the
    [n, I] intermediate rounded to bf16 once as the bf16 policy of the HIP path does."""
    res = O.moe_forward_capacity(x_cpu, w.gate.cpu(), [t.cpu() for t in w.gate_up], [t.cpu() for t in w.down],
                                 k=w.top_k, capacity_factor=w.capacity_factor,
                                 logits_override=p["logits"].cpu(), intermediate_dtype=torch.bfloat16)
    assert torch.equal(res["indices"], p["indices"].cpu().long())
    assert torch.equal(res["token_map"], p["token_map"].cpu())
    return res


def test_decode_config3_full(gpu):
    """64 tokens, H 4096, 8 experts top-2, I 14336, bf16: the whole layer against the oracle."""
    from adaptivetrainingsystem_amd import workloads as W
    w = W.make_moe_workload("c3_decode", device=gpu, gen_device="cuda")
    layer = W.build_layer(w, "fcfs")
    out, aux = layer(w.x)
    p = layer.last_plan
    ri, rw, tm, kept, dropped = _check_routing_and_plan(p, w, 64)
    _check_logits_against_own_router(p, w, w.x.reshape(-1, 4096), 64)
    assert p["capacity"] == 20
    err = _check_sampled_outputs(out, w.x.reshape(-1, 4096), w, ri, rw, tm, kept, list(range(64)), 2)
    print("config 3 full layer rel err", err, "dropped", dropped, flush=True)
    assert err <= BF16_TOL
    res = _oracle_layer(w, w.x.cpu(), p)
    assert rel_err(out, res["out"].reshape(out.shape)) <= BF16_TOL


def test_prefill_config4_full(gpu):
    """16384 tokens, Zipf-skewed logits: integer artefacts in full, every one of the 16384 output rows
    against the oracle's capacity layer (MS/core/moe_cuda_wrapper.py:413-478 restated)."""
    from adaptivetrainingsystem_amd import MoECUDAOps
    from adaptivetrainingsystem_amd import workloads as W
    w = W.make_moe_workload("c4_prefill", device=gpu, gen_device="cuda")
    layer = W.build_layer(w, "fcfs")
    out, aux = layer(w.x)
    p = layer.last_plan
    ri, rw, tm, kept, dropped = _check_routing_and_plan(p, w, 16384)
    _check_logits_against_own_router(p, w, w.x.reshape(-1, 4096), 16384)
    assert p["capacity"] == 5120 and dropped > 0 and kept.max() == 5120
    res = _oracle_layer(w, w.x.cpu(), p)
    ref = res["out"].reshape(-1, 4096)
    got = out.reshape(-1, 4096).float().cpu()
    err = rel_err(got, ref)
    # per-row bar as well: no row may hide behind the largest one
    row_err = ((got - ref).abs().amax(-1) / ref.abs().amax(-1).clamp_min(1e-3)).max().item()
    print("config 4 all 16384 rows rel err", err, "worst row", row_err, "dropped", dropped, flush=True)
    assert err <= BF16_TOL and row_err <= 2 * BF16_TOL
    # fully dropped tokens produce exact zeros
    slot = p["slot"].cpu().view(-1, 2)
    gone = (slot < 0).all(-1)
    assert gone.any() and torch.all(out.reshape(-1, 4096).cpu()[gone] == 0)
    # round trip: dispatch then combine with unit weights returns every token once per kept choice
    x_flat = w.x.reshape(-1, 4096)
    ei, tmap = MoECUDAOps.dispatch_tokens(x_flat, p["indices"], 8, 5120)
    back = MoECUDAOps.combine_expert_outputs(ei, tmap, torch.ones(16384, 2, device=gpu), 16384, 2)
    n_kept = (slot >= 0).sum(-1).to(torch.float32).to(gpu).unsqueeze(1)
    assert rel_err(back.float(), x_flat.float() * n_kept) <= 2 ** -7     # x + x is exact; one bf16 rounding


def test_finegrained_mod_config5_full(gpu):
    """16 x 2048 tokens, MoD keeps 256 per sequence, 64 experts top-6: selection and plan in full,
    every row of the block output against the oracle, skipped tokens untouched."""
    from adaptivetrainingsystem_amd import ops
    from adaptivetrainingsystem_amd import workloads as W
    w = W.make_moe_workload("c5_finegrained_mod", device=gpu, gen_device="cuda")
    block = W.build_layer(w, "fcfs")
    out, aux = block(w.x)
    scores = ops.row_dot(w.x, w.mod_weight.reshape(-1)).cpu().view(16, 2048)
    ref_scores = torch.nn.functional.linear(w.x.float().cpu(), w.mod_weight.float().cpu()).squeeze(-1)
    assert rel_err(scores, ref_scores) <= 1e-5
    sel = O.mod_select_per_sequence(scores, 256) + torch.arange(16).unsqueeze(1) * 2048
    flat = sel.reshape(-1)
    assert torch.equal(block.last_selected.cpu().long(), flat)
    p = block.moe.last_plan
    ri, rw, tm, kept, dropped = _check_routing_and_plan(p, w, 4096)
    assert p["capacity"] == 576
    gathered = w.x.reshape(-1, 2048)[flat.to(gpu)]
    _check_logits_against_own_router(p, w, gathered, 4096)
    res = _oracle_layer(w, gathered.cpu(), p)
    moe_ref = res["out"].reshape(-1, 2048)
    delta = (out.reshape(-1, 2048)[flat.to(gpu)].float() - gathered.float()).cpu()
    err = rel_err(delta, moe_ref)
    block_ref = w.x.reshape(-1, 2048).float().cpu().clone()
    block_ref[flat] += moe_ref
    block_err = rel_err(out.reshape(-1, 2048), block_ref)
    print("config 5 all 4096 kept rows rel err", err, "whole block", block_err, flush=True)
    assert err <= 2 * BF16_TOL      # delta = bf16(x + moe) - x carries the rounding of the residual sum
    assert block_err <= BF16_TOL
    untouched = torch.ones(16 * 2048, dtype=torch.bool)
    untouched[flat] = False
    assert torch.equal(out.reshape(-1, 2048).cpu()[untouched], w.x.reshape(-1, 2048).cpu()[untouched])


def test_norm_rope_config2_full(gpu):
    from adaptivetrainingsystem_amd import ops
    from adaptivetrainingsystem_amd import workloads as W
    w = W.make_norm_rope_workload(device=gpu, gen_device="cuda")
    y = ops.rmsnorm(w.x, w.norm_weight, w.eps)
    ref = O.rmsnorm(w.x.cpu(), w.norm_weight.cpu(), w.eps)
    assert rel_err(y, ref) <= 2 ** -7
    cos, sin = ops.rope_table(w.seq, w.head_dim, w.theta, device=gpu)
    rc, rs = O.rope_table(w.seq, w.head_dim, w.theta)
    assert (cos.cpu() - rc).abs().max().item() <= 1.2e-7 and (sin.cpu() - rs).abs().max().item() <= 1.2e-7
    q, k = ops.rope(w.q, w.k, cos, sin)
    rq, rk = O.rope_apply(w.q.cpu(), w.k.cpu(), cos.cpu(), sin.cpu())
    assert torch.equal(q.cpu(), rq) and torch.equal(k.cpu(), rk)
    # rotation preserves the norm of every (d, d + D/2) pair up to bf16 rounding
    def pair_norm(t):
        t = t.float()
        return t[..., :64] ** 2 + t[..., 64:] ** 2
    assert rel_err(pair_norm(q), pair_norm(w.q)) <= 4 * 2 ** -7


def test_attention_full_size_properties_and_sampled_rows(gpu):
    """Causal GQA attention at the headline shape (batch 8, seq 2048, 32 / 8 heads, head_dim 128): sampled
    query rows against the oracle, and properties that hold at any size -- doubling V doubles the output
    exactly, a prefix of the sequence gives the same rows bit for bit, a zero cotangent gives zero
    gradients, and the key gradients of V sum to the cotangent's sum (rows of P sum to one)."""
    from adaptivetrainingsystem_amd import ops
    B, Hq, Hkv, L, D = 8, 32, 8, 2048, 128
    g = torch.Generator().manual_seed(31)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    out, lse = ops.causal_attention(qg, kg, vg, return_lse=True)
    assert torch.isfinite(out.float()).all()
    # sampled (batch, head, row) triples against the oracle's row formula
    rows = torch.randint(0, L, (24,), generator=g).tolist() + [0, 1, 63, 64, 127, 128, L - 1]
    o4 = out.view(B, L, Hq, D).float().cpu()
    for n, i in enumerate(rows):
        b, h = n % B, (7 * n) % Hq
        kv = h // (Hq // Hkv)
        s = (k[b, kv, :i + 1].float() @ q[b, h, i].float()) * D ** -0.5
        p = torch.softmax(s, 0).bfloat16().float()
        ref = p @ v[b, kv, :i + 1].float()
        assert (o4[b, i, h] - ref).abs().max().item() <= BF16_TOL * max(ref.abs().max().item(), 1e-3), (b, h, i)
        assert abs(lse[b, h, i].item() - torch.logsumexp(s, 0).item()) <= 1e-3
    assert torch.equal(ops.causal_attention(qg, kg, vg * 2), out * 2)
    half = ops.causal_attention(qg[:, :, :1024], kg[:, :, :1024], vg[:, :, :1024])
    assert torch.equal(half, out[:, :1024])
    # backward
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16().to(gpu)
    dq, dk, dv = ops.causal_attention_bwd(qg, kg, vg, out, lse, dout)
    assert all(torch.isfinite(t.float()).all() for t in (dq, dk, dv))
    col = dout.view(B, L, Hkv, Hq // Hkv, D).float().sum(dim=(1, 3))          # [B, Hkv, D]
    assert rel_err(dv.float().sum(dim=2), col) <= BF16_TOL
    z = torch.zeros_like(dout)
    zq, zk, zv = ops.causal_attention_bwd(qg, kg, vg, out, lse, z)
    assert not zq.any() and not zk.any() and not zv.any()
    # sampled gradient rows: dV[j] = sum_i P[i, j] dO[i] over the queries of the group that see key j
    for n, j in enumerate([0, 5, 700, 1500, L - 1]):
        b, kv = n % B, (3 * n) % Hkv
        ref = torch.zeros(D)
        for h in range(kv * (Hq // Hkv), (kv + 1) * (Hq // Hkv)):
            s = torch.einsum("id,d->i", q[b, h, j:].float(), k[b, kv, j].float()) * D ** -0.5
            pj = torch.exp(s - lse[b, h, j:].cpu()).bfloat16().float()
            ref += pj @ dout.view(B, L, Hq, D)[b, j:, h].float().cpu()
        assert (dv[b, kv, j].float().cpu() - ref).abs().max().item() <= BF16_TOL * max(ref.abs().max().item(), 1e-3), (b, kv, j)
    # the gradients are linear in dout, and doubling is exact in every format on the way
    q2, k2, v2 = ops.causal_attention_bwd(qg, kg, vg, out, lse, dout * 2)
    assert torch.equal(q2, dq * 2) and torch.equal(k2, dk * 2) and torch.equal(v2, dv * 2)
    # sampled rows of dQ and dK from float32 arithmetic on the host:
    # dS[i, j] = P[i, j] (dO[i].V[j] - dO[i].O[i]) scale, dQ[i] = sum_j dS[i, j] K[j], dK[j] = sum_{h, i} dS[i, j] Q[i]
    out_c, lse_c, do_c = out.float().cpu().view(B, L, Hq, D), lse.cpu(), dout.float().cpu().view(B, L, Hq, D)
    scale = D ** -0.5

    def ds_block(b, h, kv, rows, cols):
        s_ = q[b, h, rows].float() @ k[b, kv, cols].float().T * scale
        p_ = torch.exp(s_ - lse_c[b, h, rows][:, None])
        p_ = torch.where(cols[None, :] <= rows[:, None], p_, torch.zeros(()))
        dp_ = do_c[b, rows, h] @ v[b, kv, cols].float().T
        dl_ = (do_c[b, rows, h] * out_c[b, rows, h]).sum(-1, keepdim=True)
        return p_ * (dp_ - dl_) * scale

    for n, i in enumerate([0, 63, 1000, L - 1]):
        b, h = (n + 1) % B, (5 * n + 2) % Hq
        kv = h // (Hq // Hkv)
        rows, cols = torch.tensor([i]), torch.arange(i + 1)
        ref = (ds_block(b, h, kv, rows, cols) @ k[b, kv, cols].float())[0]
        assert (dq[b, h, i].float().cpu() - ref).abs().max().item() <= BF16_TOL * max(ref.abs().max().item(), 1e-3), (b, h, i)
    for n, j in enumerate([0, 129, 1200, L - 1]):
        b, kv = (n + 2) % B, (3 * n + 1) % Hkv
        rows, cols = torch.arange(j, L), torch.tensor([j])
        ref = torch.zeros(D)
        for h in range(kv * (Hq // Hkv), (kv + 1) * (Hq // Hkv)):
            ref += (ds_block(b, h, kv, rows, cols).T @ q[b, h, rows].float())[0]
        assert (dk[b, kv, j].float().cpu() - ref).abs().max().item() <= BF16_TOL * max(ref.abs().max().item(), 1e-3), (b, kv, j)
