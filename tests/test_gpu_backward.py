"""Parity of the backward-pass kernels against the CPU oracle, through the C ABI.

The oracle for a gradient is what the reference computes: its explicit backward formulas for the
fused ops (restated in oracle/sparse_layer_oracle.py) and PyTorch autograd over the forward
restatement for everything else.  Bars as for the forward pass: float32 within 1e-5 and bfloat16
within 2e-2 of the oracle relative to its max-abs; the inverse rotation and the transposes are
bit-exact; float32 GEMM gradients that contract over thousands of rows get 2e-5.
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import sparse_layer_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
BF16_TOL = 2e-2


def rel_err(got, ref) -> float:
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


def tol(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.fixture(scope="module")
def ops(gpu):
    from adaptivetrainingsystem_amd import _lib, ops as _ops
    _lib.load()
    return _ops


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("shape", [(8, 512), (3, 5, 128), (7, 100), (300, 4096), (5, 8192), (3, 12000), (1, 8), (2, 6),
                                   (1000, 2048), (2500, 2048), (1, 4096), (3, 2056), (1027, 1024), (4099, 2048), (2051, 4096)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_bwd(ops, gpu, shape, dtype):
    print("case rmsnorm_bwd", shape, dtype, flush=True)
    g = gen(41)
    x = torch.randn(*shape, generator=g).to(dtype)
    dy = torch.randn(*shape, generator=g).to(dtype)
    w = torch.randn(shape[-1], generator=g) * 0.2 + 1.0
    dx_ref, dw_ref = O.rmsnorm_backward(x, w, dy, 1e-6)
    dx, dw = ops.rmsnorm_bwd(x.to(gpu), w.to(gpu), dy.to(gpu), 1e-6)
    assert dx.dtype == dtype and dx.shape == x.shape and dw.dtype == torch.float32
    assert rel_err(dx, dx_ref) <= tol(dtype)
    assert rel_err(dw, dw_ref) <= 2e-5          # float32 sums over the rows in a different order
    dx2, dw2 = ops.rmsnorm_bwd(x.to(gpu), None, dy.to(gpu), 1e-6)
    assert dw2 is None and rel_err(dx2, O.rmsnorm_backward(x, None, dy, 1e-6)[0]) <= tol(dtype)


def test_rmsnorm_bwd_bf16_weight_and_empty(ops, gpu):
    g = gen(42)
    x = torch.randn(33, 256, generator=g).bfloat16()
    dy = torch.randn(33, 256, generator=g).bfloat16()
    w = (torch.randn(256, generator=g) * 0.2 + 1.0).bfloat16()
    dx_ref, dw_ref = O.rmsnorm_backward(x, w, dy)
    dx, dw = ops.rmsnorm_bwd(x.to(gpu), w.to(gpu), dy.to(gpu))
    assert rel_err(dx, dx_ref) <= BF16_TOL and rel_err(dw, dw_ref) <= 2e-5
    e = torch.empty(0, 64, device=gpu)
    dx0, dw0 = ops.rmsnorm_bwd(e, torch.ones(64, device=gpu), e)
    assert dx0.shape == (0, 64) and torch.equal(dw0.cpu(), torch.zeros(64))


# ------------------------------------------------------------------ RoPE
@pytest.mark.parametrize("B,Hq,Hkv,L,D", [(2, 4, 2, 9, 16), (1, 16, 4, 130, 128), (2, 3, 1, 33, 64), (1, 2, 2, 5, 6)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_bwd_bit_exact(ops, gpu, B, Hq, Hkv, L, D, dtype):
    print("case rope_bwd", B, Hq, Hkv, L, D, dtype, flush=True)
    g = gen(43)
    dq = torch.randn(B, Hq, L, D, generator=g).to(dtype)
    dk = torch.randn(B, Hkv, L, D, generator=g).to(dtype)
    cos, sin = ops.rope_table(L + 7, D, half=True, device=gpu)
    rq, rk = O.rope_backward(dq, dk, cos.cpu(), sin.cpu(), position_offset=7)
    gq, gk = ops.rope(dq.to(gpu), dk.to(gpu), cos, sin, position_offset=7, inverse=True)
    assert torch.equal(gq.cpu(), rq) and torch.equal(gk.cpu(), rk)


# ------------------------------------------------------------------ silu(a) * b
@pytest.mark.parametrize("rows,cols", [(37, 1408), (5, 6), (300, 200), (1, 8), (0, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_silu_mul_fwd_bwd_on_halves(ops, gpu, rows, cols, dtype):
    print("case silu_mul", rows, cols, dtype, flush=True)
    g = gen(44)
    gu = (torch.randn(rows, 2 * cols, generator=g) * 2).to(dtype)
    dh = torch.randn(rows, cols, generator=g).to(dtype)
    a, b = gu[:, :cols].float().requires_grad_(), gu[:, cols:].float().requires_grad_()
    h_ref = F.silu(a) * b
    da_ref, db_ref = torch.autograd.grad((h_ref * dh.float()).sum(), [a, b]) if rows else (a.detach(), b.detach())
    gud = gu.to(gpu)
    h = ops.silu_mul(gud[:, :cols], gud[:, cols:])
    assert h.shape == (rows, cols) and h.dtype == dtype
    dgu = torch.empty_like(gud)
    ops.silu_mul_bwd(gud[:, :cols], gud[:, cols:], dh.to(gpu), da=dgu[:, :cols], db=dgu[:, cols:])
    if rows:
        assert rel_err(h, h_ref) <= tol(dtype)
        assert rel_err(dgu[:, :cols], da_ref) <= tol(dtype) and rel_err(dgu[:, cols:], db_ref) <= tol(dtype)
        # the dense convention of the fused wrapper (gate * silu(up)) is the same kernel with the roles swapped
        dg_ref, du_ref = O.swiglu_backward(gu[:, :cols], gu[:, cols:], dh)
        du, dg = ops.silu_mul_bwd(gud[:, cols:].contiguous(), gud[:, :cols].contiguous(), dh.to(gpu))
        assert rel_err(dg, dg_ref) <= tol(dtype) and rel_err(du, du_ref) <= tol(dtype)


# ------------------------------------------------------------------ combine
@pytest.mark.parametrize("T,E,k,C,H", [(64, 8, 2, 20, 128), (100, 4, 3, 60, 72), (512, 8, 2, 160, 512), (9, 4, 2, 2, 6)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_combine_bwd(ops, gpu, T, E, k, C, H, dtype):
    print("case combine_bwd", T, E, k, C, H, dtype, flush=True)
    g = gen(45)
    idx = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).int()
    _, token_map = O.dispatch_vectorized(torch.zeros(T, 1), idx, E, C)
    w = torch.rand(T, k, generator=g)
    y = torch.randn(E, C, H, generator=g).to(dtype)
    dout = torch.randn(T, H, generator=g).to(dtype)
    yl, wl = y.float().requires_grad_(), w.clone().requires_grad_()
    out = O.combine_vectorized(yl, token_map, wl, T, k)
    dy_ref, dw_ref = torch.autograd.grad((out * dout.float()).sum(), [yl, wl])
    dy, dw = ops.combine_bwd(dout.to(gpu), y.reshape(E * C, H).to(gpu), token_map.reshape(-1).int().to(gpu),
                             w.to(gpu), k)
    assert rel_err(dy, dy_ref.reshape(E * C, H)) <= tol(dtype)
    assert rel_err(dw, dw_ref) <= (2e-5 if dtype == torch.float32 else BF16_TOL)
    dropped = torch.ones(T * k, dtype=torch.bool)
    dropped[token_map.reshape(-1)[token_map.reshape(-1) >= 0].long()] = False
    assert torch.equal(dw.cpu().reshape(-1)[dropped], torch.zeros(int(dropped.sum())))


# ------------------------------------------------------------------ routing
@pytest.mark.parametrize("T,E,k,temp", [(300, 8, 2, 1.0), (64, 64, 6, 1.0), (50, 4, 1, 0.7), (129, 128, 4, 1.3)])
@pytest.mark.parametrize("mode", [0, 1])
def test_route_bwd(ops, gpu, T, E, k, temp, mode):
    print("case route_bwd", T, E, k, temp, mode, flush=True)
    g = gen(46)
    z = (torch.randn(T, E, generator=g) * 1.5).requires_grad_()
    noise = torch.randn(T, E, generator=g) * 0.1
    dw = torch.randn(T, k, generator=g)
    route = O.route_softmax_topk_renorm if mode == 0 else O.route_topk_softmax
    idx, w = route(z + noise, k, temp)
    aux = O.aux_loss(z, idx, E, 0.01)
    daux = 3.0
    dz_ref, = torch.autograd.grad((w * dw).sum() + aux * daux, [z])
    usage = torch.bincount(idx.reshape(-1), minlength=E).float() / (T * k + 1e-9)
    dz = ops.route_bwd((z + noise).detach().to(gpu), idx.int().to(gpu), w.detach().to(gpu), dw.to(gpu), temp, mode,
                       logits_aux=z.detach().to(gpu), usage=usage.to(gpu), aux_scale=daux * E * 0.01 / T)
    # With k = 1 the renormalised weight is p / (p + 1e-9) = 1 up to rounding: its gradient is a
    # difference of nearly equal float32 numbers (in autograd as well), so rounding noise of the order
    # eps * |dw| / tau is added to the bar.
    noise_floor = 2.5e-7 * dw.abs().max().item() / temp
    err = (dz.cpu() - dz_ref).abs().max().item()
    assert err <= 2e-5 * dz_ref.abs().max().item() + noise_floor
    # without the auxiliary term
    dz_ref2, = torch.autograd.grad((route(z + noise, k, temp)[1] * dw).sum(), [z])
    dz2 = ops.route_bwd((z + noise).detach().to(gpu), idx.int().to(gpu), w.detach().to(gpu), dw.to(gpu), temp, mode)
    assert (dz2.cpu() - dz_ref2).abs().max().item() <= 2e-5 * dz_ref2.abs().max().item() + noise_floor


@pytest.mark.parametrize("T,H,E", [(512, 512, 8), (100, 1024, 64), (33, 40, 6), (1000, 2048, 128), (1, 64, 4),
                                   (1001, 2048, 5), (300, 264, 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_bwd(ops, gpu, T, H, E, dtype):
    print("case router_bwd", T, H, E, dtype, flush=True)
    g = gen(47)
    x = torch.randn(T, H, generator=g).to(dtype)
    wg = (torch.randn(E, H, generator=g) * 0.05).to(dtype)
    dz = torch.randn(T, E, generator=g)
    base = torch.randn(T, H, generator=g).to(dtype)
    dx_ref = base.float() + dz @ wg.float()
    dw_ref = dz.T @ x.float()
    dx, dwg = ops.router_bwd(dz.to(gpu), x.to(gpu), wg.to(gpu), base=base.to(gpu))
    assert dx.dtype == dtype and rel_err(dx, dx_ref) <= tol(dtype)
    assert dwg.dtype == torch.float32 and rel_err(dwg, dw_ref) <= 2e-5
    dx0, _ = ops.router_bwd(dz.to(gpu), x.to(gpu), wg.to(gpu), need_dw=False)
    assert rel_err(dx0, dz @ wg.float()) <= tol(dtype)


# ------------------------------------------------------------------ transposes
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_transposes_exact(ops, gpu, dtype):
    g = gen(48)
    mats = [torch.randn(100, 72, generator=g).to(dtype).to(gpu) for _ in range(3)]
    outs, _ = ops.transpose_batched(mats)
    for m, o in zip(mats, outs):
        assert torch.equal(o, m.T)
    counts = torch.tensor([70, 0, 129, 64], dtype=torch.int32)
    starts = torch.tensor([0, 70, 70, 199], dtype=torch.int32)
    A, C, E = 263, 40, 4
    src = torch.randn(A, C, generator=g).to(dtype)
    ks, kc = ops.wgrad_plan(counts.to(gpu))
    assert kc.cpu().tolist() == [128, 64, 192, 64] and ks.cpu().tolist() == [0, 128, 192, 384]
    out = ops.transpose_grouped_rows(src.to(gpu), starts.to(gpu), counts.to(gpu), A)
    assert out.shape[0] == C and out.shape[1] >= 448 and out.shape[1] == ops.wgrad_padded_rows(A, E)
    ref = torch.zeros(C, 448, dtype=dtype)
    for e in range(E):
        ref[:, ks[e]:ks[e] + counts[e]] = src[starts[e]:starts[e] + counts[e]].T
    assert torch.equal(out[:, :448].cpu(), ref)
    # gathered source rows (row = table // div)
    big = torch.randn(500, C, generator=g).to(dtype)
    table = (torch.randint(0, 500, (A,), generator=g) * 2 + 1).int()
    out2 = ops.transpose_grouped_rows(big.to(gpu), starts.to(gpu), counts.to(gpu), A, gather=table.to(gpu), gather_div=2)
    gathered = big[(table // 2).long()]
    ref2 = torch.zeros(C, 448, dtype=dtype)
    for e in range(E):
        ref2[:, ks[e]:ks[e] + counts[e]] = gathered[starts[e]:starts[e] + counts[e]].T
    assert torch.equal(out2[:, :448].cpu(), ref2)


# ------------------------------------------------------------------ grouped GEMMs of the backward pass
@pytest.mark.parametrize("counts,H,I", [([70, 0, 129, 64], 128, 72), ([900, 1100], 512, 256), ([30, 20, 10, 4], 64, 136)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_expert_ffn_gradients(ops, gpu, counts, H, I, dtype):
    """gate/up pre-activation, dgrad and wgrad of the expert FFN against autograd on the oracle's expert."""
    print("case ffn grads", counts, H, I, dtype, flush=True)
    g = gen(49)
    E, A = len(counts), sum(counts)
    cnt = torch.tensor(counts, dtype=torch.int32)
    start = torch.cumsum(cnt, 0).int() - cnt
    xr = torch.randn(A, H, generator=g).to(dtype)
    wgu = [(torch.randn(2 * I, H, generator=g) * 0.05).to(dtype) for _ in range(E)]
    wd = [(torch.randn(H, I, generator=g) * 0.05).to(dtype) for _ in range(E)]
    dy = torch.randn(A, H, generator=g).to(dtype)
    # oracle: autograd over swiglu_expert per group (float32 math on the stored values)
    leaves = [t.float().requires_grad_() for t in [xr] + wgu + wd]
    ys = [O.swiglu_expert(leaves[0][start[e]:start[e] + counts[e]], leaves[1 + e], leaves[1 + E + e]) for e in range(E)]
    grads = torch.autograd.grad((torch.cat(ys) * dy.float()).sum(), leaves, allow_unused=True)
    dx_ref, dwgu_ref, dwd_ref = grads[0], grads[1:1 + E], grads[1 + E:]

    d = lambda t: t.to(gpu)
    xr_d, dy_d, cnt_d, start_d = d(xr), d(dy), d(cnt), d(start)
    wgu_d, wd_d = [d(w) for w in wgu], [d(w) for w in wd]
    tab_gu, tab_d = ops.weight_pointer_table(wgu_d), ops.weight_pointer_table(wd_d)
    # forward with saved pre-activations
    gu = ops.grouped_gemm_nt(tab_gu, H, 2 * I, start_d, cnt_d, A, A, 2 * I, H, a=xr_d)
    h = ops.silu_mul(gu[:, :I], gu[:, I:])
    y = ops.grouped_gemm_nt(tab_d, I, H, start_d, cnt_d, A, A, H, I, a=h)
    assert rel_err(y, torch.cat(ys)) <= tol(dtype)
    # dgrad
    wdT, tab_dT = ops.transpose_batched(wd_d)          # [I, H] each
    dh = ops.grouped_gemm_nt(tab_dT, H, I, start_d, cnt_d, A, A, I, H, a=dy_d)
    dgu = torch.empty_like(gu)
    ops.silu_mul_bwd(gu[:, :I], gu[:, I:], dh, da=dgu[:, :I], db=dgu[:, I:])
    wguT, tab_guT = ops.transpose_batched(wgu_d)       # [H, 2I] each
    dx = ops.grouped_gemm_nt(tab_guT, 2 * I, H, start_d, cnt_d, A, A, H, 2 * I, a=dgu)
    assert rel_err(dx, dx_ref) <= tol(dtype)
    # wgrad: one "expert" per weight matrix, K = padded rows of the expert
    ks, kc = ops.wgrad_plan(cnt_d)
    ld = ops.wgrad_padded_rows(A, E)
    es = 4 if dtype == torch.float32 else 2
    def wgrad(lhs, rhs, M, N):
        lhsT = ops.transpose_grouped_rows(lhs, start_d, cnt_d, A)     # [M, ld]
        rhsT = ops.transpose_grouped_rows(rhs, start_d, cnt_d, A)     # [N, ld]
        a_ptrs = (ks.long() * es + lhsT.data_ptr())
        b_ptrs = (ks.long() * es + rhsT.data_ptr())
        rs = torch.arange(E, dtype=torch.int32, device=gpu) * M
        rc = torch.full((E,), M, dtype=torch.int32, device=gpu)
        out = ops.grouped_gemm_nt(b_ptrs, ld, N, rs, rc, E * M, E * M, N, ld, a_ptrs=a_ptrs, lda=ld, k_count=kc,
                                  dtype=dtype, out_dtype=torch.float32)
        return out.view(E, M, N)
    dwd = wgrad(dy_d, h, H, I)
    dwgu = wgrad(dgu, xr_d, 2 * I, H)
    bar = 2e-5 if dtype == torch.float32 else BF16_TOL
    assert rel_err(dwd, torch.stack(list(dwd_ref))) <= bar
    assert rel_err(dwgu, torch.stack(list(dwgu_ref))) <= bar


# ------------------------------------------------------------------ whole layer through autograd
def _layer_grads_vs_oracle(gpu, name, capacity_mode, routing, bar, scale_tokens=None, daux=2.5, temperature=1.0,
                           overrides=None):
    """Gradients of sum(out * cot) + daux * aux w.r.t. x, the gate and every expert weight: the HIP
    autograd path against torch autograd over the oracle's forward (the reference's own training path).
    The discrete routing must coincide, which is asserted first."""
    from adaptivetrainingsystem_amd import workloads as W
    w = W.make_moe_workload(name, device="cpu", scale_tokens=scale_tokens, overrides=overrides)
    wg = W.make_moe_workload(name, device=gpu, scale_tokens=scale_tokens, overrides=overrides)
    w.routing = wg.routing = routing
    layer = W.build_layer(wg, capacity_mode)
    layer.routing_temperature = temperature
    for p in layer.parameters():
        p.requires_grad_(True)
    x = wg.x.clone().requires_grad_(True)
    out, aux = layer(x)                      # eval mode: no routing noise, gradients still flow
    assert out.requires_grad and aux.requires_grad
    g = gen(51)
    cot = torch.randn(w.x.shape, generator=g).to(w.dtype)
    (out.float() * cot.to(gpu).float()).sum().add(aux * daux).backward()

    E, k = w.num_experts, w.top_k

    def fwd(xx, wgate, *ws):
        if capacity_mode == "fcfs":
            r = O.moe_forward_capacity(xx, wgate, list(ws[:E]), list(ws[E:]), k=k, capacity_factor=w.capacity_factor,
                                       routing=routing, temperature=temperature, logit_bias=w.logit_bias)
        else:
            r = O.moe_forward_nocap(xx, wgate, list(ws[:E]), list(ws[E:]), k=k, temperature=temperature)
        fwd.last = r
        return r["out"], r["aux"]

    leaves = [w.x, w.gate] + list(w.gate_up) + list(w.down)
    grads = O.layer_grads(fwd, leaves, [cot, torch.tensor(daux)])
    # an expert that no token reached has no gradient in the oracle's autograd; here it gets zeros
    grads = [torch.zeros_like(leaf) if g_ is None else g_ for g_, leaf in zip(grads, leaves)]
    assert torch.equal(layer.last_plan["indices"].cpu().long(), fwd.last["indices"]), "routing differs from the oracle"
    if capacity_mode == "fcfs":
        assert torch.equal(layer.last_plan["token_map"].cpu(), fwd.last["token_map"])
    errs = {"x": rel_err(x.grad, grads[0]), "gate": rel_err(layer.gate.weight.grad, grads[1]),
            "gate_up": max(rel_err(ex.gate_up_proj.weight.grad, grads[2 + e]) for e, ex in enumerate(layer.experts)),
            "down": max(rel_err(ex.down_proj.weight.grad, grads[2 + E + e]) for e, ex in enumerate(layer.experts))}
    print(name, capacity_mode, routing, {n: f"{v:.2e}" for n, v in errs.items()}, flush=True)
    assert x.grad.dtype == w.dtype and layer.gate.weight.grad.dtype == w.dtype
    for n, v in errs.items():
        assert v <= bar, (n, v)


def test_layer_grads_c1_fp32(gpu):
    _layer_grads_vs_oracle(gpu, "c1_cpu_reference", "none", "softmax_topk", 2e-5)
    _layer_grads_vs_oracle(gpu, "c1_cpu_reference", "fcfs", "softmax_topk", 2e-5)
    _layer_grads_vs_oracle(gpu, "c1_cpu_reference", "fcfs", "topk_softmax", 2e-5, temperature=0.8)


def _random_layer_configs(n, seed):
    rng = np.random.default_rng(seed)
    return [(int(rng.choice([3, 40, 130, 600])), int(rng.integers(2, 9)) * 64, int(rng.choice([2, 4, 8, 16])),
             int(rng.integers(2, 4)), int(rng.integers(2, 9)) * 64, float(rng.choice([0.5, 1.25, 2.0])),
             ["fcfs", "none"][int(rng.integers(0, 2))]) for _ in range(n)]


@pytest.mark.parametrize("T,H,E,k,I,cf,mode", _random_layer_configs(8, 5))
def test_layer_grads_random_fp32_configs(gpu, T, H, E, k, I, cf, mode):
    """Every gradient of the layer on random float32 configurations (few and many rows per expert, with
    and without drops) against autograd over the oracle.  top_k >= 2: with one choice per token the
    renormalised weight is p / (p + 1e-9) = 1 to float32 rounding, its gradient is rounding noise in the
    reference's own autograd, and the gate gradient that remains (auxiliary loss only) is too small a
    yardstick for a relative bar."""
    k = min(k, E)
    ov = {"batch": 1, "seq": T, "hidden": H, "num_experts": E, "top_k": k, "intermediate": I, "capacity_factor": cf}
    print("case random layer grads", ov, mode, flush=True)
    _layer_grads_vs_oracle(gpu, "c1_cpu_reference", mode, "softmax_topk", 2e-5, overrides=ov)


def test_layer_grads_bf16_skewed_drops(gpu):
    # prefill-shaped skewed routing scaled down to 1024 tokens: expert 0 overflows its capacity
    _layer_grads_vs_oracle(gpu, "c4_prefill", "fcfs", "softmax_topk", 3e-2, scale_tokens=1024)


def test_mod_moe_block_gradients(gpu):
    """The MoD + MoE block trains: gradients of x (identity path plus the gathered rows), the gate and every
    expert against torch autograd over the oracle's composition, float32, fine-grained shape at reduced size.
    The selection is discrete, so the score weight has no gradient on either side."""
    from adaptivetrainingsystem_amd import workloads as W
    ov = {"batch": 3, "seq": 128, "hidden": 128, "intermediate": 64, "num_experts": 8, "top_k": 3, "dtype": torch.float32}
    w = W.make_moe_workload("c5_finegrained_mod", device="cpu", overrides=ov)
    wg = W.make_moe_workload("c5_finegrained_mod", device=gpu, overrides=ov)
    block = W.build_layer(wg, "fcfs")
    for p in block.moe.parameters():
        p.requires_grad_(True)
    x = wg.x.clone().requires_grad_(True)
    out, aux = block(x)
    assert out.requires_grad and aux.requires_grad
    cot = torch.randn(w.x.shape, generator=gen(61))
    (out * cot.to(gpu)).sum().add(aux * 1.5).backward()
    E, k, keep = 8, 3, int(128 * 0.125)
    sel = block.last_selected.cpu().long()
    plan = block.moe.last_plan

    def fwd(xx, wgate, *ws):
        r = O.mod_moe_block(xx, w.mod_weight, None, keep,
                            dict(gate_weight=wgate, gate_up_weights=list(ws[:E]), down_weights=list(ws[E:]), k=k,
                                 capacity_factor=w.capacity_factor, routing=wg.routing))
        fwd.last = r
        return r["block_out"], r["aux"]

    leaves = [w.x, w.gate] + list(w.gate_up) + list(w.down)
    grads = O.layer_grads(fwd, leaves, [cot, torch.tensor(1.5)])
    grads = [torch.zeros_like(leaf) if g_ is None else g_ for g_, leaf in zip(grads, leaves)]
    flat_ref = (fwd.last["selected"] + torch.arange(3).unsqueeze(1) * 128).reshape(-1)
    assert torch.equal(sel, flat_ref), "selection differs from the oracle"
    assert torch.equal(plan["indices"].cpu().long(), fwd.last["indices"]), "routing differs from the oracle"
    moe = block.moe
    errs = {"x": rel_err(x.grad, grads[0]), "gate": rel_err(moe.gate.weight.grad, grads[1]),
            "gate_up": max(rel_err(ex.gate_up_proj.weight.grad, grads[2 + e]) for e, ex in enumerate(moe.experts)),
            "down": max(rel_err(ex.down_proj.weight.grad, grads[2 + E + e]) for e, ex in enumerate(moe.experts))}
    print("mod block grads", {n: f"{v:.2e}" for n, v in errs.items()}, flush=True)
    for n, v in errs.items():
        assert v <= 2e-5, (n, v)
    # rows the block skipped get exactly the cotangent (identity path only)
    skipped = torch.ones(3 * 128, dtype=torch.bool)
    skipped[sel] = False
    assert torch.equal(x.grad.reshape(-1, 128).cpu()[skipped], cot.reshape(-1, 128)[skipped])
    assert block.router.weight.grad is None


def test_training_mode_noise_and_stats(gpu):
    """Training mode: noise on the routing logits only; the auxiliary loss still uses the clean logits."""
    from adaptivetrainingsystem_amd import workloads as W
    wg = W.make_moe_workload("c1_cpu_reference", device=gpu)
    layer = W.build_layer(wg, "none")
    for p in layer.parameters():
        p.requires_grad_(True)
    layer.train()
    layer.noise_std = 0.5
    torch.manual_seed(7)
    out, aux = layer(wg.x)
    plan = layer.last_plan
    ref_aux = O.aux_loss(plan["logits"].cpu(), plan["indices"].cpu().long(), wg.num_experts, layer.load_balancing_weight)
    assert abs(aux.item() - ref_aux.item()) <= 1e-6
    clean_idx = O.route_softmax_topk_renorm(plan["logits"].cpu(), wg.top_k)[0]
    assert (clean_idx != plan["indices"].cpu().long()).any(), "noise of 0.5 should change some routing decision"
    (out.sum() + aux).backward()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in layer.parameters())
    stats = layer.get_routing_stats()
    assert stats["total_tokens_routed"] == wg.tokens
    # the no-grad path of the same layer takes the auxiliary loss from the clean logits too: same seed, same noise
    for p in layer.parameters():
        p.requires_grad_(False)
    torch.manual_seed(7)
    with torch.no_grad():
        out2, aux2 = layer(wg.x)
    assert torch.equal(layer.last_plan["indices"], plan["indices"])
    assert abs(aux2.item() - aux.item()) <= 1e-7
    assert (out2 - out).abs().max().item() <= 1e-5 * out.abs().max().item()


def test_module_gradients_norm_rope_expert_swiglu(gpu):
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.seams.cuda_opt_wrapper import FusedSwiGLU
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    g = gen(52)
    # RMSNorm module
    norm = A.RMSNorm(256).to(gpu)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(256, generator=g) * 0.2 + 1)
    x = torch.randn(4, 9, 256, generator=g)
    dy = torch.randn(4, 9, 256, generator=g)
    xg = x.to(gpu).requires_grad_()
    norm(xg).backward(dy.to(gpu))
    dx_ref, dw_ref = O.rmsnorm_backward(x, norm.weight.detach().cpu(), dy)
    assert rel_err(xg.grad, dx_ref) <= F32_TOL and rel_err(norm.weight.grad, dw_ref) <= 2e-5
    # rotary embedding through apply_rotary_pos_emb
    rot = A.RotaryEmbedding(32, max_seq_len=64)
    cos, sin = rot(17, gpu)
    q = torch.randn(2, 4, 17, 32, generator=g)
    k = torch.randn(2, 2, 17, 32, generator=g)
    qg, kg = q.to(gpu).requires_grad_(), k.to(gpu).requires_grad_()
    qo, ko = A.apply_rotary_pos_emb(qg, kg, cos, sin)
    dq, dk = torch.randn(2, 4, 17, 32, generator=g), torch.randn(2, 2, 17, 32, generator=g)
    torch.autograd.backward([qo, ko], [dq.to(gpu), dk.to(gpu)])
    rq, rk = O.rope_backward(dq, dk, cos.cpu(), sin.cpu())
    assert torch.equal(qg.grad.cpu(), rq) and torch.equal(kg.grad.cpu(), rk)
    # one expert
    ex = A.SwiGLUExpert(LayerConfig(128, 72, 1, 1)).to(gpu)
    xe = torch.randn(50, 128, generator=g)
    de = torch.randn(50, 128, generator=g)
    xeg = xe.to(gpu).requires_grad_()
    ex(xeg).backward(de.to(gpu))
    grads = O.layer_grads(lambda a, b, c: O.swiglu_expert(a, b, c),
                          [xe, ex.gate_up_proj.weight.detach().cpu(), ex.down_proj.weight.detach().cpu()], [de])
    assert rel_err(xeg.grad, grads[0]) <= 2e-5
    assert rel_err(ex.gate_up_proj.weight.grad, grads[1]) <= 2e-5 and rel_err(ex.down_proj.weight.grad, grads[2]) <= 2e-5
    # dense SwiGLU block of the fused wrapper (gate * silu(up))
    blk = FusedSwiGLU(64, 96).to(gpu)
    xs = torch.randn(10, 64, generator=g)
    ds = torch.randn(10, 96, generator=g)
    xsg = xs.to(gpu).requires_grad_()
    blk(xsg).backward(ds.to(gpu))
    wgp, wup = blk.gate_proj.weight.detach().cpu(), blk.up_proj.weight.detach().cpu()
    ref = O.layer_grads(lambda a, b, c: (a @ b.T) * F.silu(a @ c.T), [xs, wgp, wup], [ds])
    assert rel_err(xsg.grad, ref[0]) <= 2e-5 and rel_err(blk.gate_proj.weight.grad, ref[1]) <= 2e-5


# ------------------------------------------------------------------ trainer-facing management
def test_trainer_surgery_and_checkpoint_round_trip(gpu):
    """What the reference trainer does to a live layer between steps (add_expert / prune_expert /
    adjust_capacity_factor / adjust_routing_temperature, trainer.py:1269-1493) and a state_dict round trip:
    after every change forward and backward still agree with the oracle on the layer's current weights."""
    import torch.nn as nn
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd import workloads as W
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    torch.manual_seed(11)
    cfg = LayerConfig(128, 72, 4, 2, 1.25, moe_routing="softmax_topk", moe_capacity_mode="fcfs")
    layer = A.MoEFFNLayer(cfg).to(gpu)
    layer.eval()
    g = gen(53)
    x = torch.randn(3, 50, 128, generator=g)
    cot = torch.randn(3, 50, 128, generator=g)

    def check():
        xg = x.to(gpu).requires_grad_()
        for p in layer.parameters():
            p.grad = None
        out, aux = layer(xg)
        (out * cot.to(gpu)).sum().add(aux).backward()
        E = layer.num_experts
        ws = [layer.gate.weight] + [ex.gate_up_proj.weight for ex in layer.experts] + \
             [ex.down_proj.weight for ex in layer.experts]

        def fwd(xx, wgate, *rest):
            r = O.moe_forward_capacity(xx, wgate, list(rest[:E]), list(rest[E:]), k=layer.top_k,
                                       capacity_factor=layer.capacity_factor, temperature=layer.routing_temperature)
            fwd.last = r
            return r["out"], r["aux"]

        grads = O.layer_grads(fwd, [x] + [w_.detach().cpu() for w_ in ws], [cot, torch.tensor(1.0)])
        assert torch.equal(layer.last_plan["indices"].cpu().long(), fwd.last["indices"])
        assert layer.last_plan["capacity"] == fwd.last["capacity"]
        assert rel_err(out, fwd.last["out"]) <= F32_TOL
        assert rel_err(xg.grad, grads[0]) <= 2e-5
        for w_, g_ in zip(ws, grads[1:]):
            assert rel_err(w_.grad, g_) <= 2e-5
        return out.detach()

    check()
    # add_expert: average of the existing experts plus noise, gate row appended, new nn.Linear gate
    new = A.SwiGLUExpert(cfg).to(gpu)
    with torch.no_grad():
        for name, p in new.named_parameters():
            p.copy_(torch.stack([dict(e.named_parameters())[name] for e in layer.experts]).mean(0))
            p.add_(torch.randn_like(p) * 0.01)
    layer.experts.append(new)
    layer.num_experts += 1
    old = layer.gate.weight.data
    grown = torch.zeros(layer.num_experts, 128, device=gpu)
    grown[:-1] = old
    nn.init.normal_(grown[-1], mean=0.0, std=0.01)
    layer.gate = nn.Linear(128, layer.num_experts, bias=False).to(gpu)
    layer.gate.weight.data = grown
    layer.train()                      # statistics follow the new expert count
    layer.noise_std = 0.0
    check()
    assert len(layer.get_routing_stats()["expert_usage_percentages"]) == 5
    layer.eval()
    # adjust_capacity_factor / adjust_routing_temperature
    layer.capacity_factor = 0.6
    layer.routing_temperature = 1.7
    check()
    assert int((layer.last_plan["hist"] - layer.last_plan["kept"]).sum()) > 0       # the tighter capacity drops
    # prune_expert
    del layer.experts[1]
    layer.num_experts -= 1
    w_old = layer.gate.weight.data
    layer.gate = nn.Linear(128, layer.num_experts, bias=False).to(gpu)
    layer.gate.weight.data = torch.cat([w_old[:1], w_old[2:]], dim=0)
    before = check()
    # checkpoint round trip: the reference's key names, loaded into a fresh layer
    sd = {k_: v.cpu() for k_, v in layer.state_dict().items()}
    assert set(sd) == {"gate.weight"} | {f"experts.{i}.{n}.weight" for i in range(4) for n in ("gate_up_proj", "down_proj")}
    fresh = A.MoEFFNLayer(cfg).to(gpu).eval()
    fresh.load_state_dict(sd)
    fresh.capacity_factor, fresh.routing_temperature = layer.capacity_factor, layer.routing_temperature
    with torch.no_grad():
        again, _ = fresh(x.to(gpu))
    assert torch.equal(again, before)
