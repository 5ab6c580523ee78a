"""Seeded random shapes through the attention and K-sliced product paths, against the CPU oracle.  The fixed
cases elsewhere pin known edges; these sweep the shape space around them (tile remainders, head ratios, cache
lengths on both sides of the thresholds that switch kernels)."""
import os

import numpy as np
import pytest
import torch

from oracle import sparse_layer_oracle as O

pytestmark = pytest.mark.gpu
BF16_TOL = 2e-2
# ATS_RANDOM_SCALE=10 runs ten times as many cases from the same generators (a deeper sweep by hand)
SCALE = max(1, int(os.environ.get("ATS_RANDOM_SCALE", "1")))


def rel_err(got, ref) -> float:
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


def _attention_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        D = int(rng.choice([64, 128]))
        Hkv = int(rng.choice([1, 2, 3, 4]))
        Hq = Hkv * int(rng.choice([1, 2, 4, 8]))
        B = int(rng.integers(1, 4))
        regime = rng.integers(0, 3)
        if regime == 0:      # prefill, no cache
            L = int(rng.integers(1, 500)); Lk = L
        elif regime == 1:    # a chunk on top of a cache
            L = int(rng.integers(1, 200)); Lk = L + int(rng.integers(1, 900))
        else:                # decoding: few rows, long cache (key ranges)
            L = int(rng.integers(1, 5)); Lk = L + int(rng.integers(200, 1500))
        cases.append((B, Hq, Hkv, L, Lk, D, bool(rng.integers(0, 2))))
    return cases


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D,masked", _attention_cases(36 * SCALE, 2024))
def test_attention_random_shapes(gpu, B, Hq, Hkv, L, Lk, D, masked):
    from adaptivetrainingsystem_amd import ops
    print("case random attention", B, Hq, Hkv, L, Lk, D, masked, flush=True)
    g = torch.Generator().manual_seed(B * 1000003 + Hq * 10007 + L * 101 + Lk)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    mask = None
    if masked:      # right padding that leaves every query a real key, plus a padded stretch inside
        mask = torch.ones(B, Lk)
        for b in range(B):
            n_real = int(torch.randint(Lk - L + 1, Lk + 1, (1,), generator=g))
            mask[b, n_real:] = 0
        if Lk - L > 40:
            mask[:, 10:30] = 0
    rep = Hq // Hkv
    q32, k32, v32 = (t.float().requires_grad_() for t in (q, k, v))
    ref = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5, mask)
    ref.backward(dout.float())
    bias = None if mask is None else ((1.0 - mask) * -1e4).to(gpu)
    out, lse = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), return_lse=True, key_bias=bias)
    assert rel_err(out, ref) <= BF16_TOL
    dq, dk, dv = ops.causal_attention_bwd(q.to(gpu), k.to(gpu), v.to(gpu), out, lse, dout.to(gpu), key_bias=bias)
    assert rel_err(dv, v32.grad) <= BF16_TOL
    assert rel_err(dq, q32.grad) <= BF16_TOL
    assert rel_err(dk, k32.grad) <= BF16_TOL


def _linear_cases(n, seed):
    rng = np.random.default_rng(seed)
    return [(int(rng.integers(1, 300)), int(rng.integers(1, 40)) * 8, int(rng.integers(1, 48)) * 64,
             [torch.float32, torch.bfloat16][int(rng.integers(0, 2))]) for _ in range(n)]


@pytest.mark.parametrize("T,N,K,dtype", _linear_cases(24 * SCALE, 7))
def test_linear_random_shapes(gpu, T, N, K, dtype):
    """Few rows against a weight matrix: plain and K-sliced tilings, whichever the shape selects."""
    from adaptivetrainingsystem_amd import ops
    print("case random linear", T, N, K, dtype, ops.down_k_splits(1, T, N, K, dtype), flush=True)
    g = torch.Generator().manual_seed(T * 7919 + N * 31 + K)
    x = torch.randn(T, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    got = ops.linear_nt(x.to(gpu), w.to(gpu))
    assert rel_err(got, x.double() @ w.double().T) <= (1e-5 if dtype == torch.float32 else BF16_TOL)


def _kmajor_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        E = int(rng.integers(1, 7))
        counts = [int(c) for c in rng.integers(0, 900, E)]
        counts[int(rng.integers(0, E))] += 193 * E        # the K-major kernel serves groups above 192 rows on average
        K = int(rng.integers(1, 17)) * 64
        N = int(rng.integers(1, 150)) * 8
        pad = int(rng.choice([0, 0, 8, 64]))
        cases.append((counts, K, N, pad, bool(rng.integers(0, 2)), bool(rng.integers(0, 2))))
    return cases


@pytest.mark.parametrize("counts,K,N,pad,gather,f32_out", _kmajor_cases(16 * SCALE, 23))
def test_kmajor_product_random_shapes(gpu, counts, K, N, pad, gather, f32_out):
    """Grouped product against weights stored [K, N] (row stride N + pad): float64 reference and the bits of the NT
    product against a transposed copy, over random group sizes, tile remainders in N, K from one slab upwards."""
    from adaptivetrainingsystem_amd import ops
    print("case random k-major", counts, K, N, pad, gather, f32_out, flush=True)
    E, n = len(counts), sum(counts)
    g = torch.Generator().manual_seed(n * 31 + K * 7 + N)
    ldb = N + pad
    store = [(torch.randn(K, ldb, generator=g) * 0.05).bfloat16().to(gpu) for _ in range(E)]
    w = [x[:, :N] for x in store]                                   # [K, N] views with row stride ldb
    wT = [x.t().contiguous() for x in w]
    tab = torch.tensor([x.data_ptr() for x in store], dtype=torch.int64, device=gpu)
    tabT = ops.weight_pointer_table(wT)
    count = torch.tensor(counts, dtype=torch.int32)
    start = (torch.cumsum(count, 0) - count).to(torch.int32).to(gpu)
    count = count.to(gpu)
    src_rows = n + 5
    a = torch.randn(src_rows, K, generator=g).bfloat16().to(gpu)
    rows = torch.randint(0, 3 * src_rows, (n,), generator=g).to(torch.int32).to(gpu) if gather else None
    a_used = a[(rows // 3).long()] if gather else a[:n]
    out_dtype = torch.float32 if f32_out else torch.bfloat16
    assert ops.grouped_gemm_nn_supported(E, n, N, K, ldb, torch.bfloat16)
    out = ops.grouped_gemm_nn(tab, ldb, start, count, n, n, N, K, a, a_rows=rows, a_row_div=3, out_dtype=out_dtype)
    ref = ops.grouped_gemm_nt(tabT, K, N, start, count, n, n, N, K, a=a_used.contiguous(), out_dtype=out_dtype)
    assert torch.equal(out, ref)
    off = 0
    for e, c in enumerate(counts):
        if c:
            r64 = a_used[off:off + c].cpu().double() @ w[e].cpu().double()
            assert rel_err(out[off:off + c], r64) <= BF16_TOL
        off += c


def _layer_cases(n, seed):
    rng = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        E = int(rng.choice([2, 4, 8, 16, 64]))
        k = int(rng.integers(1, min(E, 6) + 1))
        H = int(rng.integers(2, 17)) * 64
        I = int(rng.integers(2, 17)) * 64
        T = int(rng.choice([1, 3, 17, 64, 130, 300, 700, 1500]))
        cf = float(rng.choice([0.5, 1.0, 1.25, 2.0]))
        dtype = [torch.float32, torch.bfloat16][int(rng.integers(0, 2))]
        mode = ["fcfs", "none"][int(rng.integers(0, 2))]
        cases.append((T, H, E, k, I, cf, dtype, mode))
    return cases


@pytest.mark.parametrize("T,H,E,k,I,cf,dtype,mode", _layer_cases(20 * SCALE, 11))
def test_moe_layer_random_configs(gpu, T, H, E, k, I, cf, dtype, mode):
    """The whole MoE layer on random small configurations (decode-size, mid-size and prefill tiles, sliced
    and plain down projections, drops and no drops): integers bit for bit, output to the float bar."""
    from adaptivetrainingsystem_amd import workloads as W
    print("case random layer", T, H, E, k, I, cf, dtype, mode, flush=True)
    ov = {"batch": 1, "seq": T, "hidden": H, "num_experts": E, "top_k": k, "intermediate": I, "capacity_factor": cf,
          "dtype": dtype, "zipf_bias": 0.0}
    w = W.make_moe_workload("c1_cpu_reference", device="cpu", overrides=ov)
    wg = W.make_moe_workload("c1_cpu_reference", device=gpu, overrides=ov)
    layer = W.build_layer(wg, mode)
    out, aux = layer(wg.x)
    p = layer.last_plan
    logits_gpu = p["logits"].cpu()
    kw = dict(k=k, temperature=1.0, logits_override=logits_gpu)
    if mode == "fcfs":
        ref = O.moe_forward_capacity(w.x, w.gate, w.gate_up, w.down, capacity_factor=cf, routing="softmax_topk", **kw)
        assert p["capacity"] == ref["capacity"]
        assert torch.equal(p["token_map"].cpu(), ref["token_map"]) and torch.equal(p["slot"].cpu(), ref["slot"])
        assert torch.equal(p["kept"].cpu().long(), ref["kept"])
    else:
        ref = O.moe_forward_nocap(w.x, w.gate, w.gate_up, w.down, **kw)
    assert torch.equal(p["indices"].cpu().long(), ref["indices"])
    assert (p["weights"].cpu() - ref["weights"]).abs().max().item() <= 1e-5
    assert rel_err(out, ref["out"]) <= (1e-5 if dtype == torch.float32 else BF16_TOL)
    assert abs(aux.item() - ref["aux"].item()) <= 1e-6
