"""Parity of the gfx950 HIP path against the CPU oracle, through the C ABI.

Bars: integer artefacts (expert indices, histograms, slots, token maps,
permutation tables, selections) bit-exact; float32 outputs within 1e-5 of the
oracle relative to the oracle's max-abs; bfloat16 outputs within 2e-2 on the
same measure (the kernels accumulate in float32 and round once per tensor).
Routing is compared bit-exactly on bit-equal logits: the oracle is fed the
logits the GPU produced, and the logits themselves are compared separately
with the float bar.
"""
import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import sparse_layer_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
BF16_TOL = 2e-2


def rel_err(got: torch.Tensor, ref: torch.Tensor) -> float:
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


def gen(seed):
    return torch.Generator().manual_seed(seed)


def same_bits(got: torch.Tensor, ref: torch.Tensor) -> bool:
    got, ref = got.detach().cpu(), ref.detach().cpu()
    if got.shape != ref.shape or got.dtype != ref.dtype:
        print("shape/dtype differ", got.shape, ref.shape, got.dtype, ref.dtype, flush=True)
        return False
    if torch.equal(got, ref):
        return True
    d = (got.double() - ref.double()).abs()
    print(f"{int((d > 0).sum())} of {d.numel()} elements differ, max abs {d.max().item():.3e}, first at "
          f"{(d > 0).nonzero()[:4].tolist()}", flush=True)
    return False


@pytest.fixture(scope="module")
def A(gpu):
    import adaptivetrainingsystem_amd as pkg
    from adaptivetrainingsystem_amd import _lib
    _lib.load()
    return pkg


@pytest.fixture(scope="module")
def ops(A):
    from adaptivetrainingsystem_amd import ops as _ops
    return _ops


def test_calibration_yardsticks_move_the_bytes_they_claim(gpu):
    """The streaming copy copies exactly, the streaming read leaves its sink alone (ragged sizes included)."""
    from adaptivetrainingsystem_amd import profiling
    g = torch.Generator(device=gpu)
    g.manual_seed(11)
    for n in (16, 4096 + 16, 3 * 1024 * 1024 + 48):
        src = torch.randint(0, 255, (n,), dtype=torch.uint8, device=gpu, generator=g)
        dst = torch.zeros_like(src)
        profiling.stream_copy(src, dst)
        assert torch.equal(src, dst)
        sink = torch.full((16,), 7, dtype=torch.uint8, device=gpu)
        profiling.stream_read(src, sink)
        torch.cuda.synchronize()
        assert bool((sink == 7).all())


# ------------------------------------------------------------------ RMSNorm
@pytest.mark.parametrize("shape", [(8, 512), (3, 5, 128), (7, 100), (64, 4096), (5, 8192), (3, 12000), (1, 8),
                                   (1000, 2048)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm(ops, gpu, shape, dtype):
    print("case rmsnorm", shape, dtype, flush=True)
    x = (torch.randn(*shape, generator=gen(1)) * 1.7).to(dtype)
    w = 1 + 0.1 * torch.randn(shape[-1], generator=gen(2))
    ref = O.rmsnorm(x, w, 1e-6)
    got = ops.rmsnorm(x.to(gpu), w.to(gpu), 1e-6)
    assert got.dtype == dtype and got.shape == x.shape
    assert rel_err(got, ref) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)
    if dtype == torch.bfloat16:   # stricter: at most one bf16 ulp from the oracle's rounding
        assert rel_err(got, ref) <= 2 ** -7
    got_now = ops.rmsnorm(x.to(gpu), None, 1e-6)
    assert rel_err(got_now, O.rmsnorm(x, None, 1e-6)) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)


def test_rmsnorm_bf16_weight_extremes_and_empty(ops, gpu):
    x = torch.randn(16, 256, generator=gen(3)).bfloat16()
    w = (1 + 0.1 * torch.randn(256, generator=gen(4))).bfloat16()
    assert rel_err(ops.rmsnorm(x.to(gpu), w.to(gpu)), O.rmsnorm(x, w)) <= 2 ** -7
    for s in (1e-6, 1e6):     # the reference's own stability case
        xs = torch.randn(2, 10, 128, generator=gen(5)) * s
        got = ops.rmsnorm(xs.to(gpu), torch.ones(128, device=gpu))
        assert torch.isfinite(got).all()
        assert rel_err(got, O.rmsnorm(xs, torch.ones(128))) <= F32_TOL
    assert ops.rmsnorm(torch.empty(0, 64, device=gpu), None).shape == (0, 64)


def test_rmsnorm_module_api(A, gpu):
    m = A.RMSNorm(96).to(gpu)
    x = torch.randn(2, 10, 96, generator=gen(6))
    with torch.no_grad():
        m.weight.copy_(1 + 0.1 * torch.randn(96, generator=gen(7)))
    assert rel_err(m(x.to(gpu)), O.rmsnorm(x, m.weight.cpu())) <= F32_TOL
    f = A.FusedRMSNorm(96).to(gpu)
    assert rel_err(f(x.to(gpu)), O.rmsnorm(x, torch.ones(96))) <= F32_TOL
    with pytest.raises(A.AtsError):
        m(x)                      # CPU tensor: no fallback


# ------------------------------------------------------------------ RoPE
@pytest.mark.parametrize("L,D,scaling", [(300, 64, None), (2048, 128, None), (64, 32, 2.0), (17, 6, None)])
def test_rope_table(ops, gpu, L, D, scaling):
    cos, sin = ops.rope_table(L, D, 10000.0, scaling, device=gpu)
    rc, rs = O.rope_table(L, D, 10000.0, scaling)
    assert cos.shape == (L, D)
    assert (cos.cpu() - rc).abs().max().item() <= 1.2e-7
    assert (sin.cpu() - rs).abs().max().item() <= 1.2e-7
    ch, sh = ops.rope_table(L, D, 10000.0, scaling, half=True, device=gpu)
    assert torch.equal(ch, cos[:, : D // 2]) and torch.equal(sh, sin[:, : D // 2])


@pytest.mark.parametrize("B,Hq,Hkv,L,D", [(2, 4, 2, 9, 16), (1, 16, 4, 130, 128), (2, 3, 1, 33, 64), (1, 2, 2, 5, 6),
                                          (1, 5, 1, 70, 256), (2, 8, 8, 64, 32)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rope_apply_bit_exact(ops, gpu, B, Hq, Hkv, L, D, dtype):
    print("case rope", B, Hq, Hkv, L, D, dtype, flush=True)
    q = torch.randn(B, Hq, L, D, generator=gen(8)).to(dtype)
    k = torch.randn(B, Hkv, L, D, generator=gen(9)).to(dtype)
    cos, sin = O.rope_table(L, D)
    rq, rk = O.rope_apply(q, k, cos, sin)
    gq, gk = ops.rope(q.to(gpu), k.to(gpu), cos.to(gpu), sin.to(gpu))
    assert gq.dtype == dtype
    # products and sums are rounded separately on both sides: identical bits
    assert same_bits(gq, rq) and same_bits(gk, rk)


def test_rope_strided_inputs_and_fused_module(A, ops, gpu):
    B, L, Hq, Hkv, D = 2, 40, 8, 2, 64
    qs = torch.randn(B, L, Hq, D, generator=gen(10))
    ks = torch.randn(B, L, Hkv, D, generator=gen(11))
    q, k = qs.transpose(1, 2), ks.transpose(1, 2)          # [B,H,L,D] views, as the attention layer makes them
    rope = A.RotaryEmbedding(D, max_seq_len=16)
    cos, sin = rope(L, gpu)                                # forces a cache extension
    assert cos.shape == (L, D) and rope.max_seq_len >= L
    rq, rk = O.rope_apply(q, k, *O.rope_table(L, D))
    gq, gk = A.apply_rotary_pos_emb(qs.to(gpu).transpose(1, 2), ks.to(gpu).transpose(1, 2), cos, sin)
    assert gq.is_contiguous() and rel_err(gq, rq) <= 1e-6 and rel_err(gk, rk) <= 1e-6
    fused = A.FusedRoPE(D, max_seq_len=128)
    off = 7
    gq2, gk2 = fused(q.contiguous().to(gpu), k.contiguous().to(gpu), position_offset=off)
    ch, sh = fused.cos_cache.cpu(), fused.sin_cache.cpu()
    rq2, rk2 = O.fused_rope_apply(q, k, ch, sh, off)
    assert same_bits(gq2, rq2) and same_bits(gk2, rk2)
    with pytest.raises(A.AtsError):
        fused(q.contiguous().to(gpu), k.contiguous().to(gpu), position_offset=128)   # beyond the table


# ------------------------------------------------------------------ router GEMM
@pytest.mark.parametrize("T,H,E", [(512, 512, 8), (100, 1024, 64), (33, 40, 6), (1, 4096, 8), (257, 2048, 128),
                                   (64, 200, 8),
                                   # the instances chosen at the benchmark shapes: the flat kernel (>= 2048 tokens,
                                   # <= 16 experts), whose 8 waves each walk a full 4-step K slice at H 4096, and
                                   # the 4-wave kernel for 33-64 experts
                                   (2048, 4096, 8), (16384, 4096, 8), (4096, 2048, 16), (4096, 2048, 64),
                                   (32768, 2048, 64), (2049, 4096, 5), (3000, 1000, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_router_logits(ops, gpu, T, H, E, dtype):
    print("case router", T, H, E, dtype, flush=True)
    x = torch.randn(T, H, generator=gen(12)).to(dtype)
    w = (torch.randn(E, H, generator=gen(13)) * 0.02).to(dtype)
    ref = x.double() @ w.double().T
    got = ops.router_logits(x.to(gpu), w.to(gpu))
    assert got.dtype == torch.float32 and got.shape == (T, E)
    assert rel_err(got, ref) <= F32_TOL
    assert rel_err(got, O.router_logits(x, w)) <= F32_TOL
    bias = torch.randn(E, generator=gen(14))
    assert rel_err(ops.router_logits(x.to(gpu), w.to(gpu), bias.to(gpu)), ref + bias.double()) <= F32_TOL


# ------------------------------------------------------------------ routing
def _ambiguous_rows(logits, k, temperature):
    """Rows where two of the top-(k+1) tempered logits are equal: selection order is then a
    library property of torch.topk, not of the algorithm."""
    s = torch.sort(logits / temperature, dim=-1, descending=True)[0][:, : k + 1]
    return (s[:, :-1] == s[:, 1:]).any(-1)


@pytest.mark.parametrize("T,E,k,temp", [(512, 8, 2, 1.0), (1000, 64, 6, 1.0), (37, 4, 1, 1.0), (300, 128, 4, 0.7),
                                        (129, 6, 3, 1.3), (16384, 8, 2, 1.0), (50, 300, 8, 1.0), (700, 40, 5, 0.8),
                                        (4096, 64, 6, 1.0), (333, 33, 16, 1.0), (500, 24, 4, 1.1), (40, 20, 3, 1.0),
                                        (900, 12, 2, 0.9), (10, 50, 7, 1.0)])
def test_route_topk(ops, gpu, T, E, k, temp):
    print("case route", T, E, k, temp, flush=True)
    logits = torch.randn(T, E, generator=gen(15)) * 1.3
    amb = _ambiguous_rows(logits, k, temp)
    assert amb.sum().item() <= max(1, T // 1000)
    for variant, oracle_fn in ((0, O.route_softmax_topk_renorm), (1, O.route_topk_softmax)):
        r = ops.route_topk(logits.to(gpu), k, temp, variant, load_balancing_weight=0.01)
        ri, rw = oracle_fn(logits, k, temp)
        gi = r["indices"].cpu().long()
        assert gi.dtype == torch.int64 and torch.equal(gi[~amb], ri[~amb])
        assert (r["weights"].cpu()[~amb] - rw[~amb]).abs().max().item() <= 1e-5
        hist = torch.bincount(gi.reshape(-1), minlength=E)
        assert torch.equal(r["hist"].cpu().long(), hist)
        colsum = torch.softmax(logits.double(), -1).sum(0)
        assert rel_err(r["prob_colsum"], colsum) <= 1e-5
        aux_ref = O.aux_loss(logits, gi, E, 0.01)
        assert abs(r["aux"].item() - aux_ref.item()) <= 1e-6


def test_route_topk_ties_go_to_lower_index(ops, gpu):
    logits = torch.tensor([[1.0, 1.0, 1.0, 1.0, 0.5, 1.0, 0.0, 1.0], [0.0, 2.0, 2.0, -1.0, 2.0, 0.0, 0.0, 0.0]])
    r = ops.route_topk(logits.to(gpu), 2, 1.0, 1, with_stats=False)
    assert r["indices"].cpu().tolist() == [[0, 1], [1, 2]]
    assert torch.allclose(r["weights"].cpu(), torch.full((2, 2), 0.5))


def test_route_topk_one_token_per_wave_order(ops, gpu):
    """33..64 experts and more than 64 tokens take the kernel that selects with wave-wide reductions of an
    unsigned key: ties go to the lower index, -0 equals +0, NaN ranks first, -inf last."""
    T, E, k = 200, 64, 6
    logits = torch.randn(T, E, generator=gen(151))
    logits[0, :] = 1.0                                  # all equal: experts 0..5
    logits[1, 10:20] = 7.0                              # ten equal maxima: 10..15
    logits[2, :] = -1.0
    logits[2, 5], logits[2, 9], logits[2, 40] = 0.0, -0.0, 0.0      # zeros of both signs tie: 5, 9, 40, then 0, 1, 2
    logits[3, 17] = float("nan")                        # NaN first
    logits[3, 3] = float("inf")
    logits[4, :] = float("-inf")
    logits[4, 60:] = torch.tensor([0.5, 0.25, 0.5, 0.125])           # 60, 62, 61, 63, then -inf ties 0, 1
    r = ops.route_topk(logits.to(gpu), k, 1.0, 1, with_stats=False)
    idx = r["indices"].cpu().tolist()
    assert idx[0] == [0, 1, 2, 3, 4, 5]
    assert idx[1] == [10, 11, 12, 13, 14, 15]
    assert idx[2] == [5, 9, 40, 0, 1, 2]
    assert idx[3][:2] == [17, 3]
    assert idx[4] == [60, 62, 61, 63, 0, 1]
    # every other row: the order of a stable sort by descending value
    ref = torch.sort(logits[5:], dim=-1, descending=True, stable=True)[1][:, :k]
    assert torch.equal(r["indices"].cpu().long()[5:], ref)


def test_topk_gating_api(A, gpu):
    logits = torch.randn(64, 8, generator=gen(16))
    idx, w = A.MoECUDAOps.topk_gating(logits.to(gpu), 2, temperature=0.5)
    ri, rw = O.route_topk_softmax(logits, 2, 0.5)
    assert idx.dtype == torch.int64 and torch.equal(idx.cpu(), ri)
    assert (w.cpu() - rw).abs().max().item() <= 1e-5


# ------------------------------------------------------------------ dispatch plan
def _check_plan(ops, gpu, idx, E, C, idx_dtype=torch.int32):
    T, k = idx.shape
    plan = ops.dispatch_plan(idx.to(idx_dtype).to(gpu), E, C)
    tm, slot, hist, kept, dropped = c_oracle.fcfs_dispatch(idx.numpy(), E, C)
    assert plan["status"].item() == 0
    assert np.array_equal(plan["slot"].cpu().numpy(), slot)
    assert np.array_equal(plan["token_map"].cpu().numpy(), tm)
    assert np.array_equal(plan["hist"].cpu().numpy(), hist)
    assert np.array_equal(plan["kept"].cpu().numpy(), kept)
    offsets = np.concatenate([[0], np.cumsum(kept)]).astype(np.int32)
    assert np.array_equal(plan["offsets"].cpu().numpy(), offsets)
    total = int(offsets[-1])
    row_src = plan["row_src"].cpu().numpy()
    expect_src = np.concatenate([tm[e, : kept[e]] for e in range(E)]) if total else np.zeros(0, np.int32)
    assert np.array_equal(row_src[:total], expect_src)
    assert (row_src[total:] == -1).all()
    row_of = plan["row_of"].cpu().numpy()
    expect_of = np.full(T * k, -1, np.int32)
    expect_of[expect_src] = np.arange(total, dtype=np.int32)
    assert np.array_equal(row_of, expect_of)
    assert total + dropped == T * k
    return plan


@pytest.mark.parametrize("T,E,k,C", [(16, 4, 2, 5), (512, 8, 2, 160), (64, 8, 2, 20), (300, 8, 3, 0), (1500, 8, 2, 1000000 // 8),
                                     (4096, 64, 6, 576), (16384, 8, 2, 5120), (32768, 64, 6, 4608), (700, 300, 4, 7),
                                     # the one-launch form (1025 .. 32768 assignments): ragged ends, replica counts
                                     (513, 8, 2, 100), (3001, 5, 3, 2000), (10922, 20, 3, 1500), (8000, 70, 4, 600),
                                     (16385, 8, 2, 5120)])
def test_dispatch_plan_bit_exact(ops, gpu, T, E, k, C):
    print("case plan", T, E, k, C, flush=True)
    g = gen(17 + T)
    skew = torch.log(1.0 / torch.arange(1, E + 1).float()) * 1.5
    idx = torch.topk(torch.randn(T, E, generator=g) + skew, k, -1)[1]
    C = min(C, T * k)
    _check_plan(ops, gpu, idx, E, C)
    _check_plan(ops, gpu, idx, E, C, torch.int64)


def test_dispatch_plan_special_cases(ops, gpu):
    _check_plan(ops, gpu, torch.zeros(3000, 1, dtype=torch.int64), 4, 100)          # everything to one expert
    _check_plan(ops, gpu, torch.tensor([[0, 1], [0, 2], [0, 1], [1, 2]]), 3, 2)    # hand-worked case of the oracle tests
    bad = torch.tensor([[0, 9], [1, 2]], dtype=torch.int32)
    assert ops.dispatch_plan(bad.to(gpu), 4, 2)["status"].item() == 1


def test_dispatch_tokens_and_combine_api(A, gpu):
    T, H, E, k, C = 96, 40, 8, 2, 20
    g = gen(18)
    x = torch.randn(T, H, generator=g)
    idx = torch.topk(torch.randn(T, E, generator=g), k, -1)[1]
    w = torch.softmax(torch.randn(T, k, generator=g), -1)
    ei_ref, tm_ref = O.dispatch_loop(x, idx, E, C)
    ei, tm = A.MoECUDAOps.dispatch_tokens(x.to(gpu), idx.to(gpu), E, C)
    assert tm.dtype == torch.int32 and torch.equal(tm.cpu(), tm_ref) and torch.equal(ei.cpu(), ei_ref)
    eo = torch.randn(E, C, H, generator=g)
    out_ref = O.combine_loop(eo, tm_ref, w, T, k)
    out = A.MoECUDAOps.combine_expert_outputs(eo.to(gpu), tm, w.to(gpu), T, k)
    assert same_bits(out, out_ref)          # float32, same order, separately rounded: identical bits
    xb = x.bfloat16()
    eib, _ = A.MoECUDAOps.dispatch_tokens(xb.to(gpu), idx.to(gpu), E, C)
    assert torch.equal(eib.cpu(), O.dispatch_loop(xb, idx, E, C)[0])
    H2 = 37                                         # odd width: scalar paths
    x2 = torch.randn(T, H2, generator=g)
    ei2, tm2 = A.MoECUDAOps.dispatch_tokens(x2.to(gpu), idx.to(gpu), E, C)
    assert torch.equal(ei2.cpu(), O.dispatch_loop(x2, idx, E, C)[0])
    eo2 = torch.randn(E, C, H2, generator=g)
    out2 = A.MoECUDAOps.combine_expert_outputs(eo2.to(gpu), tm2, w.to(gpu), T, k)
    assert same_bits(out2, O.combine_loop(eo2, tm_ref, w, T, k))


@pytest.mark.parametrize("T,H,E,k,C", [(50, 260, 8, 2, 20), (40, 64, 16, 12, 40), (30, 6, 4, 3, 30), (20, 516, 8, 2, 3),
                                       (33, 1030, 16, 9, 25)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_combine_scalar_path_tail_columns(A, gpu, T, H, E, k, C, dtype):
    """Widths and k values that take the scalar combine kernel (H not a multiple of 8, or more than 8 choices),
    with a last trip of the column loop that only the first lanes make: every column against the literal loop
    (MS/core/moe_cuda_wrapper.py:328-359)."""
    g = gen(180 + H)
    idx = torch.topk(torch.randn(T, E, generator=g), k, -1)[1]
    w = torch.softmax(torch.randn(T, k, generator=g), -1)
    _, tm_ref = O.dispatch_loop(torch.zeros(T, 1), idx, E, C)
    eo = torch.randn(E, C, H, generator=g).to(dtype)
    ref = O.combine_loop(eo.float(), tm_ref, w, T, k)
    out = A.MoECUDAOps.combine_expert_outputs(eo.to(gpu), tm_ref.to(gpu), w.to(gpu), T, k)
    assert out.dtype == dtype
    if dtype == torch.float32:
        assert same_bits(out, ref)
    else:
        assert torch.equal(out.cpu(), ref.bfloat16())       # float32 sums in the same order, one rounding


# ------------------------------------------------------------------ expert FFN (grouped GEMMs)
@pytest.mark.parametrize("n,H,I", [(20, 512, 1408), (70, 512, 1408), (300, 256, 200), (1000, 512, 384), (33, 72, 136),
                                   (1, 64, 64), (2500, 128, 256), (8, 1024, 512), (1, 2048, 256), (32, 4096, 128)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu_expert_single_group(A, gpu, n, H, I, dtype):
    print("case expert", n, H, I, dtype, flush=True)
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    ex = A.SwiGLUExpert(LayerConfig(H, I, 1, 1))
    g = gen(19)
    with torch.no_grad():
        ex.gate_up_proj.weight.copy_(torch.randn(2 * I, H, generator=g) * 0.05)
        ex.down_proj.weight.copy_(torch.randn(H, I, generator=g) * 0.05)
    ex = ex.to(dtype)
    x = torch.randn(n, H, generator=g).to(dtype)
    ref = O.swiglu_expert(x, ex.gate_up_proj.weight, ex.down_proj.weight)
    got = ex.to(gpu)(x.to(gpu))
    assert got.dtype == dtype and got.shape == (n, H)
    assert rel_err(got, ref) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)


def test_grouped_gateup_gather_small_and_huge_source(ops, gpu):
    """The fused gather must give the same bits as a GEMM over pre-gathered rows, both when the
    source fits 32-bit lane offsets (direct-to-LDS kernel) and when it does not (a 4.4 GB source
    tensor, which selects the 64-bit-pointer kernel)."""
    print("case gather paths", flush=True)
    H, I, n = 512, 256, 1100
    g = gen(23)
    w = (torch.randn(2 * I, H, generator=g) * 0.05).bfloat16().to(gpu)
    tab = ops.weight_pointer_table([w])
    start = torch.zeros(1, dtype=torch.int32, device=gpu)
    count = torch.full((1,), n, dtype=torch.int32, device=gpu)
    rows_small = torch.randn(n, H, generator=g).bfloat16().to(gpu)
    base = ops.grouped_gateup_swiglu(rows_small, tab, start, count, n, n, H, I)
    ref = O.swiglu_expert(rows_small.cpu(), w.cpu(), torch.zeros(H, I, dtype=torch.bfloat16))  # shape check only
    assert base.shape == (n, I) and ref.shape == (n, H)
    for total_rows in (5000, 4_400_000):          # 5 MB and 4.5 GB of source rows
        src = torch.empty(total_rows, H, dtype=torch.bfloat16, device=gpu)
        idx = torch.randperm(n, generator=g).to(gpu) * (total_rows // n) + (total_rows // n - 1)
        src[idx] = rows_small
        k = 2
        a_rows = (idx * k + 1).to(torch.int32)     # row index = a_rows // k
        got = ops.grouped_gateup_swiglu(src, tab, start, count, n, n, H, I, a_rows=a_rows, a_row_div=k)
        assert same_bits(got, base), f"gather from {total_rows} rows"
        del src


@pytest.mark.parametrize("counts,H,I,S", [([19, 17, 0, 14, 17, 1, 17, 13], 512, 1024, 2), ([5, 48, 20], 256, 2048, 4),
                                          ([33], 384, 4096, 8), ([1, 0, 2, 48], 128, 512, 1), ([200, 3, 97], 256, 1024, 2)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grouped_down_split_along_k(ops, gpu, counts, H, I, S, dtype):
    """Decode-size down projection cut into S slices of K: the partial results add up to the unsplit
    product (float32: to rounding of the sum order; against the float64 product with the float bar), rows
    outside the groups are never written, and the combine over partial results gives the same bits as
    the combine over their rounded sum."""
    print("case split k", counts, H, I, S, dtype, flush=True)
    g = gen(61)
    E, rows = len(counts), sum(counts)
    h = (torch.randn(rows, I, generator=g) * 0.5).to(dtype)
    wd = [(torch.randn(H, I, generator=g) * 0.05).to(dtype) for _ in range(E)]
    off = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    start = torch.tensor(off[:-1], dtype=torch.int32, device=gpu)
    count = torch.tensor(counts, dtype=torch.int32, device=gpu)
    wd_gpu = [w.to(gpu) for w in wd]
    tab = ops.weight_pointer_table(wd_gpu)
    parts = ops.grouped_down_splitk(h.to(gpu), tab, start, count, rows, H, I, S)
    assert parts.shape == (S, rows, H) and parts.dtype == torch.float32
    ref = torch.cat([h[off[e]:off[e + 1]].double() @ wd[e].double().T for e in range(E)])
    y32 = ops.sum_partials(parts, torch.float32)
    assert rel_err(y32, ref) <= (F32_TOL if dtype == torch.float32 else 1e-5)
    unsplit = ops.grouped_down(h.to(gpu), tab, start, count, rows, H, I, out_dtype=torch.float32)
    assert rel_err(y32, unsplit) <= 1e-5
    y = ops.sum_partials(parts, dtype)
    assert rel_err(y, ref) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)
    # combine: two choices per token drawn from the rows
    T, k = 11, 2
    row_of = torch.randint(-1, rows, (T * k,), generator=g, dtype=torch.int32)
    for t in range(T):                                   # a token does not visit a row twice
        if row_of[2 * t] == row_of[2 * t + 1]:
            row_of[2 * t + 1] = -1
    w = torch.rand(T, k, generator=g)
    res = torch.randn(T, H, generator=g).to(dtype)
    for residual in (None, res.to(gpu)):
        a = ops.combine_partials(parts, row_of.to(gpu), w.to(gpu), T, k, dtype, residual=residual)
        b = ops.combine(y, row_of.to(gpu), w.to(gpu), T, k, out_dtype=dtype, residual=residual)
        assert same_bits(a, b)


@pytest.mark.parametrize("T,N,K", [(1, 4096, 4096), (8, 1024, 2048), (48, 512, 1536), (17, 264, 1000), (64, 2048, 4096),
                                   (200, 1024, 2048), (300, 512, 1024)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_nt_few_rows(ops, gpu, T, N, K, dtype):
    """A few rows against a whole weight matrix (decode): the K-sliced path (several 32-row tiles from 33
    rows on) and, where K does not slice (1000 columns) or there are more than 256 rows, the plain one."""
    print("case linear few rows", T, N, K, dtype, flush=True)
    g = gen(62)
    x = torch.randn(T, K, generator=g).to(dtype)
    w = (torch.randn(N, K, generator=g) * 0.05).to(dtype)
    got = ops.linear_nt(x.to(gpu), w.to(gpu))
    assert got.shape == (T, N) and got.dtype == dtype
    assert rel_err(got, x.double() @ w.double().T) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)
    expect_split = T <= 256 and K % 128 == 0
    assert (ops.down_k_splits(1, T, N, K, dtype) > 1) == expect_split


# ------------------------------------------------------------------ whole layer
def _layer_vs_oracle(A, gpu, name, capacity_mode, routing, tol, scale_tokens=None, overrides=None, temperature=1.0):
    from adaptivetrainingsystem_amd import workloads as W
    w = W.make_moe_workload(name, device="cpu", scale_tokens=scale_tokens, overrides=overrides)
    w.routing = routing
    wg = W.make_moe_workload(name, device=gpu, scale_tokens=scale_tokens, overrides=overrides)
    wg.routing = routing
    layer = W.build_layer(wg, capacity_mode)
    layer.routing_temperature = temperature
    out, aux = layer(wg.x)
    p = layer.last_plan
    logits_gpu = p["logits"].cpu()
    kw = dict(k=w.top_k, temperature=temperature, logits_override=logits_gpu)
    if capacity_mode == "fcfs":
        ref = O.moe_forward_capacity(w.x, w.gate, w.gate_up, w.down, capacity_factor=w.capacity_factor,
                                     routing=routing, **kw)
        assert p["capacity"] == ref["capacity"]
        assert torch.equal(p["token_map"].cpu(), ref["token_map"])
        assert torch.equal(p["slot"].cpu(), ref["slot"])
        assert torch.equal(p["kept"].cpu().long(), ref["kept"])
    else:
        assert routing == "softmax_topk"
        ref = O.moe_forward_nocap(w.x, w.gate, w.gate_up, w.down, **kw)
        assert (p["slot"] >= 0).all()
    # logits: float bar against the oracle's own router
    own = O.router_logits(w.x.reshape(-1, w.hidden), w.gate)
    if w.logit_bias is not None:
        own = own + w.logit_bias.cpu()
    assert rel_err(logits_gpu, own) <= F32_TOL
    # routing on bit-equal logits: identical integers
    assert torch.equal(p["indices"].cpu().long(), ref["indices"])
    assert (p["weights"].cpu() - ref["weights"]).abs().max().item() <= 1e-5
    assert torch.equal(p["hist"].cpu().long(), torch.bincount(ref["indices"].reshape(-1), minlength=w.num_experts))
    assert out.shape == w.x.shape and out.dtype == w.dtype
    err = rel_err(out, ref["out"])
    assert err <= tol, err
    assert abs(aux.item() - ref["aux"].item()) <= 1e-6
    # how many tokens would route differently on the oracle's own logits (reported, expected 0 or near-ties)
    own_idx = O.route_softmax_topk_renorm(own, w.top_k, temperature)[0]
    mism = (own_idx != ref["indices"]).any(-1).sum().item()
    print(f"{name}/{capacity_mode}/{routing}: out rel err {err:.3e}, rows routed differently on oracle logits: {mism}",
          flush=True)
    assert mism <= max(1, w.tokens // 500)
    return p, ref


def test_layer_c1_fp32_capacity(A, gpu):
    """Config 1 at full size: 512 tokens, H 512, 8 experts top-2, I 1408, cf 1.25, float32, after RMSNorm."""
    from adaptivetrainingsystem_amd import workloads as W
    p, ref = _layer_vs_oracle(A, gpu, "c1_cpu_reference", "fcfs", "softmax_topk", F32_TOL)
    assert p["capacity"] == 160
    # the pre-norm pipeline of the config: out = MoE(RMSNorm(x))
    w = W.make_moe_workload("c1_cpu_reference", device="cpu")
    wg = W.make_moe_workload("c1_cpu_reference", device=gpu)
    norm = A.RMSNorm(512).to(gpu)
    layer = W.build_layer(wg, "fcfs")
    xn = norm(wg.x)
    out, aux = layer(xn)
    xn_ref = O.rmsnorm(w.x, torch.ones(512))
    assert rel_err(xn, xn_ref) <= F32_TOL
    r = O.moe_forward_capacity(xn.cpu(), w.gate, w.gate_up, w.down, k=2, capacity_factor=1.25,
                               logits_override=layer.last_plan["logits"].cpu())
    assert torch.equal(layer.last_plan["token_map"].cpu(), r["token_map"])
    assert rel_err(out, r["out"]) <= F32_TOL


def test_layer_c1_variants(A, gpu):
    _layer_vs_oracle(A, gpu, "c1_cpu_reference", "none", "softmax_topk", F32_TOL)
    _layer_vs_oracle(A, gpu, "c1_cpu_reference", "fcfs", "topk_softmax", F32_TOL, temperature=0.8)
    _layer_vs_oracle(A, gpu, "c1_cpu_reference", "fcfs", "softmax_topk", BF16_TOL,
                     overrides={"dtype": torch.bfloat16})
    # forcing many drops
    p, ref = _layer_vs_oracle(A, gpu, "c1_cpu_reference", "fcfs", "softmax_topk", F32_TOL,
                              overrides={"capacity_factor": 0.5})
    assert (p["slot"] < 0).sum().item() > 0


def test_layer_decode_shaped_bf16(A, gpu):
    """Config 3's shape class (64 tokens, weight-streaming small groups) at reduced H/I so that the
    CPU oracle's weights stay small."""
    p, _ = _layer_vs_oracle(A, gpu, "c3_decode", "fcfs", "softmax_topk", BF16_TOL,
                            overrides={"hidden": 1024, "intermediate": 2048})
    assert p["capacity"] == 20


def test_layer_prefill_shaped_skewed_bf16(A, gpu):
    """Config 4's shape class (Zipf-skewed logits, overflowing experts, 256-row tiles) at reduced size."""
    p, _ = _layer_vs_oracle(A, gpu, "c4_prefill", "fcfs", "softmax_topk", BF16_TOL, scale_tokens=8192,
                            overrides={"hidden": 512, "intermediate": 1024})
    dropped = (p["slot"] < 0).sum().item()
    print("dropped assignments:", dropped, flush=True)
    assert dropped > 0 and p["kept"].cpu().max().item() == p["capacity"]


def test_mod_moe_block_c5_shaped(A, ops, gpu):
    """Config 5's composition (MoD top-12.5% per sequence -> gather -> 64-expert top-6 MoE -> scatter-add)
    at reduced size; each piece compared with the oracle."""
    from adaptivetrainingsystem_amd import workloads as W
    ov = {"batch": 4, "seq": 512, "hidden": 256, "intermediate": 128}
    w = W.make_moe_workload("c5_finegrained_mod", device="cpu", overrides=ov)
    wg = W.make_moe_workload("c5_finegrained_mod", device=gpu, overrides=ov)
    block = W.build_layer(wg, "fcfs")
    out, aux = block(wg.x)
    keep = int(512 * 0.125)
    scores_gpu = ops.row_dot(wg.x, wg.mod_weight.reshape(-1)).cpu().view(4, 512)
    scores_ref = torch.nn.functional.linear(w.x.float(), w.mod_weight.float()).squeeze(-1)
    assert rel_err(scores_gpu, scores_ref) <= F32_TOL
    sel_ref = O.mod_select_per_sequence(scores_gpu, keep)                  # selection on bit-equal scores
    flat_ref = (sel_ref + torch.arange(4).unsqueeze(1) * 512).reshape(-1)
    assert torch.equal(block.last_selected.cpu().long(), flat_ref)
    gathered = w.x.reshape(-1, 256)[flat_ref]
    p = block.moe.last_plan
    ref = O.moe_forward_capacity(gathered, w.gate, w.gate_up, w.down, k=6, capacity_factor=1.5,
                                 routing=wg.routing, logits_override=p["logits"].cpu())
    assert p["capacity"] == O.capacity(4 * keep, 6, 64, 1.5)
    assert torch.equal(p["indices"].cpu().long(), ref["indices"])
    assert torch.equal(p["token_map"].cpu(), ref["token_map"])
    expect = w.x.reshape(-1, 256).float().clone()
    expect[flat_ref] += ref["out"].reshape(-1, 256)
    assert rel_err(out.reshape(-1, 256), expect) <= BF16_TOL
    untouched = torch.ones(4 * 512, dtype=torch.bool)
    untouched[flat_ref] = False
    assert torch.equal(out.reshape(-1, 256).cpu()[untouched], w.x.reshape(-1, 256)[untouched])


def test_mod_router_eval_and_selection(A, ops, gpu):
    m = A.MoDRouter(64, capacity_factor=0.5, routing_temperature=0.9).to(gpu).eval()
    with torch.no_grad():
        m.router.weight.copy_(torch.randn(1, 64, generator=gen(20)) * 0.3)
        m.router.bias.fill_(0.1)
    x = torch.randn(3, 50, 64, generator=gen(21))
    mask, probs, aux = m(x.to(gpu))
    pr = O.mod_router_probs(x, m.router.weight.cpu(), m.router.bias.cpu(), 0.9)
    assert aux is None and mask.shape == (3, 50, 1)
    assert (probs.cpu() - pr).abs().max().item() <= 1e-6
    assert torch.equal(mask.cpu(), O.mod_router_eval_mask(probs.cpu(), 0.5))     # threshold on bit-equal probs
    st = m.get_routing_stats()                          # MS/core/model.py:990-995, 998-1011
    assert st["total_tokens_routed"] == 150 and st["computed_tokens"] == mask.sum().item() == 76
    assert st["skipped_tokens"] == 74 and abs(st["compute_ratio"] + st["skip_ratio"] - 1) < 1e-12
    m(x.to(gpu))
    assert m.get_routing_stats()["computed_tokens"] == 152
    m.reset_routing_stats()
    assert "error" in m.get_routing_stats()
    s = torch.randn(5, 700, generator=gen(22))
    s[0, 10] = s[0, 3]                                                           # a tie
    sel = ops.select_topk_per_sequence(s.to(gpu), 77).cpu().view(5, 77)
    ref = O.mod_select_per_sequence(s, 77) + torch.arange(5).unsqueeze(1) * 700
    assert torch.equal(sel.long(), ref)


def _lowest_index_topk_mask(v, k):
    """Exactly k ones at the k largest values; among equal values the lower index first."""
    order = torch.sort(-v.double(), stable=True)[1][:k]
    m = torch.zeros_like(v)
    m[order] = 1.0
    return m


@pytest.mark.parametrize("n,k", [(150, 75), (1, 1), (1, 0), (1000, 0), (1000, 1000), (1000, 1500), (5000, 1), (16383, 4000),
                                 (16384, 8192), (70000, 123), (524288, 65536)])
def test_topk_mask_ste_exact_count_and_ties(ops, gpu, n, k):
    """The mask of the MoD router's training branch: exactly min(k, n) ones, at the largest values, the lower
    index first among equals (one workgroup up to 16383 values, digit passes over many workgroups above);
    heavy ties, a tie that straddles the threshold, signed zeros and infinities; and the straight-through
    weights (mask - v) + v bit for bit."""
    print("case topk_mask", n, k, flush=True)
    g = gen(400 + n % 97 + k % 13)
    kk = min(k, n)
    cases = [torch.rand(n, generator=g)]
    tied = torch.randint(0, 5, (n,), generator=g).float() * 0.25            # five distinct values
    cases.append(tied)
    half = torch.rand(n, generator=g)
    half[::3] = 0.5                                                         # a third of the values are equal
    cases.append(half)
    sgn = torch.randn(n, generator=g)
    sgn[::5] = 0.0
    sgn[1::5] = -0.0
    if n > 10:
        sgn[2], sgn[7] = float("inf"), float("-inf")
    cases.append(sgn)
    for v in cases:
        mask, ste = ops.topk_mask_ste(v.to(gpu), k)
        want = _lowest_index_topk_mask(v, kk)
        assert int(mask.sum().item()) == kk
        assert torch.equal(mask.cpu(), want)
        fin = torch.isfinite(v)
        assert torch.equal(ste.cpu()[fin], ((want - v) + v)[fin])
        assert torch.equal(ops.topk_mask_ste(v.to(gpu), k, want_ste=False).cpu(), want)


def test_mod_router_training_branch(A, ops, gpu):
    """MoDRouter in training mode (MS/core/model.py:941-965) against the oracle's restatement: probabilities,
    mask (on bit-equal probabilities), straight-through weights, auxiliary loss, statistics, and the gradients of
    x, the router weight and the bias under a per-token cotangent on both outputs."""
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 2e-2)):
        m = A.MoDRouter(96, capacity_factor=0.3, routing_temperature=1.7).to(gpu).train()
        with torch.no_grad():
            m.router.weight.copy_(torch.randn(1, 96, generator=gen(51)) * 0.3)
            m.router.bias.fill_(-0.2)
        x = torch.randn(4, 70, 96, generator=gen(52)).to(dtype)
        cw = torch.randn(4, 70, 1, generator=gen(53))
        cp = torch.randn(4, 70, 1, generator=gen(54))
        xg = x.to(gpu).requires_grad_()
        weights, probs, aux = m(xg)
        assert weights.shape == probs.shape == (4, 70, 1) and weights.dtype == torch.float32
        xr = x.float().requires_grad_()
        wr = m.router.weight.detach().cpu().to(dtype).float().requires_grad_()
        br = m.router.bias.detach().cpu().clone().requires_grad_()
        rw, rp, rmask, raux = O.mod_router_train(xr, wr, br, 1.7, 0.3)
        assert (probs.detach().cpu() - rp.detach()).abs().max().item() <= (2e-6 if dtype == torch.float32 else 2e-6)
        k = int(280 * 0.3)
        mask_gpu = (weights.detach() > 0.5).float().cpu()
        assert int(mask_gpu.sum()) == k
        assert torch.equal(mask_gpu.view(-1), _lowest_index_topk_mask(probs.detach().cpu().view(-1), k))   # bit-equal probs
        differs = int((mask_gpu != rmask).sum())
        assert differs <= 2                         # only a near-tie of the two sets of probabilities may differ
        assert (weights.detach().cpu() - mask_gpu).abs().max().item() <= 1.2e-7
        assert abs(aux.item() - raux.item()) <= 1e-7 and not aux.requires_grad
        st = m.get_routing_stats()
        assert st["total_tokens_routed"] == 280 and st["computed_tokens"] == k and st["skipped_tokens"] == 280 - k
        torch.autograd.backward([weights, probs], [cw.to(gpu), cp.to(gpu)])
        torch.autograd.backward([rw, rp], [cw, cp])
        assert rel_err(xg.grad, xr.grad) <= tol
        assert rel_err(m.router.weight.grad, wr.grad) <= max(tol, 2e-5)
        assert rel_err(m.router.bias.grad, br.grad) <= 2e-5
        # capacity_factor >= 1: every token computed, weights of one, zero auxiliary loss
        m2 = A.MoDRouter(96, capacity_factor=1.0).to(gpu).train()
        w2, _, aux2 = m2(x.to(gpu))
        assert (w2 - 1.0).abs().max().item() <= 1.2e-7 and aux2.item() == 0.0


def test_dense_swiglu_with_mod_trains(A, gpu):
    """DenseSwiGLUWithMoD (MS/core/model.py:1304-1403) in training mode: the FFN output of every token times
    its straight-through routing weight; output and all gradients against the oracle's pieces."""
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    torch.manual_seed(23)
    cfg = LayerConfig(128, 256, 1, 1, use_mod=True, mod_capacity_factor=0.5, mod_routing_temperature=1.0)
    ffn = A.DenseSwiGLUWithMoD(cfg)
    with torch.no_grad():
        ffn.gate_up_proj.weight.mul_(6.0)
        ffn.down_proj.weight.mul_(6.0)
        ffn.router.router.weight.copy_(torch.randn(1, 128, generator=gen(55)) * 0.2)
    ffn = ffn.to(gpu).train()
    x = torch.randn(2, 48, 128, generator=gen(56))
    dy = torch.randn(2, 48, 128, generator=gen(57))
    xg = x.to(gpu).requires_grad_()
    out, aux = ffn(xg)
    out.backward(dy.to(gpu))
    p = {n: t.detach().cpu().clone().requires_grad_() for n, t in ffn.named_parameters()}
    xr = x.clone().requires_grad_()
    rw, _, rmask, raux = O.mod_router_train(xr, p["router.router.weight"], p["router.router.bias"], 1.0, 0.5)
    ref = O.swiglu_expert(xr, p["gate_up_proj.weight"], p["down_proj.weight"]) * rw
    ref.backward(dy)
    assert int((out.detach().abs().amax(-1) > 0).sum()) == 48          # half of the 96 tokens are computed
    assert rel_err(out, ref) <= 1e-5 and abs(aux.item() - raux.item()) <= 1e-7
    assert rel_err(xg.grad, xr.grad) <= 2e-5
    for n, t in ffn.named_parameters():
        assert t.grad is not None and rel_err(t.grad, p[n].grad) <= 3e-5, n
    # evaluation mode keeps the threshold branch
    ffn.eval()
    with torch.no_grad():
        out_e, aux_e = ffn(x.to(gpu))
    assert aux_e is None and torch.isfinite(out_e).all()


@pytest.mark.parametrize("L,keep", [(513, 1), (700, 700), (2048, 256), (2049, 300), (3000, 1), (4096, 4000),
                                    (8192, 1024)])
def test_select_topk_long_sequences_with_ties(ops, gpu, L, keep):
    """Sequences above 512 positions take the radix-select kernel: heavy ties (scores from a handful of values),
    signed zeros (equal scores) and infinities against the stable-sort oracle."""
    g = gen(300 + L)
    B = 3
    s = torch.randn(B, L, generator=g)
    s[1] = torch.randint(-2, 3, (L,), generator=g).float() * 0.5           # five distinct values, zeros included
    s[1, ::7] = -0.0
    s[2, : L // 3] = float("inf")
    s[2, L // 3: L // 2] = float("-inf")
    s[0, 5] = s[0, 400]
    sel = ops.select_topk_per_sequence(s.to(gpu), keep).cpu().view(B, keep)
    ref = O.mod_select_per_sequence(s, keep) + torch.arange(B).unsqueeze(1) * L
    assert torch.equal(sel.long(), ref)


@pytest.mark.parametrize("aligned", [0, 1])
@pytest.mark.parametrize("counts,BM,n_tiles,SM,SN,slices", [
    ([5120, 4000, 300, 0, 1, 256, 257, 77], 256, 112, 4, 8, 1),
    ([384] * 64, 256, 11, 8, 4, 1),
    ([7, 0, 300, 129] * 40, 128, 5, 4, 8, 1),            # 160 groups: three 64-group steps of the search
    ([20, 16, 0, 3] * 20, 32, 40, 1, 32, 2),             # 80 experts x 2 K slices
])
def test_tile_schedule_on_device_equals_host(gpu, counts, BM, n_tiles, SM, SN, slices, aligned):
    """The wave-parallel search of the GEMM kernels (prefix scan by shuffles, ballot, 64 groups per step) gives
    every block id the tile that the sequential host walk gives it."""
    from adaptivetrainingsystem_amd import _lib
    lib = _lib.load()
    rc = np.asarray(counts, dtype=np.int32)
    E = len(counts)
    blocks = lib.ats_debug_grid_blocks(int(rc.sum()) * slices, E * slices, BM, n_tiles, SM, SN, aligned)
    out = torch.full((blocks, 4), -7, dtype=torch.int32, device=gpu)
    rc_dev = torch.from_numpy(rc).to(gpu)
    assert lib.ats_debug_decode_tiles_device(rc_dev.data_ptr(), E, BM, n_tiles, SM, SN, aligned, slices, blocks,
                                             out.data_ptr(), None) == 0
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    want = np.full((blocks, 4), -1, dtype=np.int32)
    o4 = np.zeros(4, dtype=np.int32)
    for b in range(blocks):
        if lib.ats_debug_decode_tile(b, rc.ctypes.data, E, BM, n_tiles, SM, SN, aligned, slices, o4.ctypes.data):
            want[b] = o4
    assert (want[:, 0] >= 0).sum() == slices * n_tiles * sum(-(-c // BM) for c in counts)
    assert np.array_equal(got, want)


def test_fused_rmsnorm_float32_output(A, gpu):
    """The reference's fused wrapper returns float32 for any input dtype (cuda_opt_wrapper.py:91-117); the module
    follows the input dtype unless asked for that behaviour."""
    x = torch.randn(5, 7, 96, generator=gen(61)).bfloat16()
    w = 1.0 + 0.1 * torch.randn(96, generator=gen(62))
    ref32 = O.rmsnorm(x.float(), w, 1e-6)
    plain = A.FusedRMSNorm(96).to(gpu)
    legacy = A.FusedRMSNorm(96, float32_output=True).to(gpu)
    with torch.no_grad():
        plain.weight.copy_(w)
        legacy.weight.copy_(w)
        y_plain, y_legacy = plain(x.to(gpu)), legacy(x.to(gpu))
    assert y_plain.dtype == torch.bfloat16 and y_legacy.dtype == torch.float32
    assert (y_legacy.cpu() - ref32).abs().max().item() <= 1e-5 * ref32.abs().max().item()
    assert (y_plain.float().cpu() - ref32).abs().max().item() <= 2 ** -7 * ref32.abs().max().item()


def test_performance_monitor_api(A, gpu):
    """The monitor of the reference's operator module (moe_cuda_wrapper.py:76-159, 599-611): same keys, fed by HIP
    events instead of synchronisations, only while it is switched on."""
    from adaptivetrainingsystem_amd import profiling as P
    P.reset_performance_monitor()
    assert P.get_performance_summary() == {"status": "No data yet"}
    logits = torch.randn(300, 8, generator=gen(41)).to(gpu)
    A.MoECUDAOps.topk_gating(logits, 2)
    assert P.get_performance_summary() == {"status": "No data yet"}          # off by default
    P.enable_performance_monitor(True)
    try:
        idx, w = A.MoECUDAOps.topk_gating(logits, 2)
        A.MoECUDAOps.dispatch_tokens(torch.randn(300, 64, generator=gen(42)).to(gpu), idx, 8, 100)
    finally:
        P.enable_performance_monitor(False)
    st = P.get_performance_summary()
    assert set(st) == {"cuda_calls", "pytorch_calls", "cuda_time_ms", "pytorch_time_ms", "cuda_percentage",
                       "estimated_speedup", "tokens_per_sec_cuda", "tokens_per_sec_pytorch"}
    assert st["cuda_calls"] == 2 and st["pytorch_calls"] == 0 and st["cuda_time_ms"] > 0
    assert st["cuda_percentage"] == 100 and st["tokens_per_sec_cuda"] > 0
    m = P.MoEPerformanceMonitor()
    m.record_cuda(2.0, 100)
    m.record_pytorch(6.0, 100)
    assert m.get_stats()["estimated_speedup"] == 3.0 and m.get_stats()["tokens_per_sec_pytorch"] == 100 / 0.006
    # a loop that monitors and never asks for statistics holds a bounded number of events
    P.reset_performance_monitor()
    P.enable_performance_monitor(True)
    try:
        small = torch.randn(16, 8, generator=gen(43)).to(gpu)
        for _ in range(1500):
            A.MoECUDAOps.topk_gating(small, 2)
    finally:
        P.enable_performance_monitor(False)
    assert len(P._GLOBAL_MONITOR._pending) <= P.MoEPerformanceMonitor._PENDING_BOUND + 1
    st = P.get_performance_summary()
    assert st["cuda_calls"] == 1500 and st["cuda_time_ms"] > 0 and not P._GLOBAL_MONITOR._pending
    P.reset_performance_monitor()


def test_fused_swiglu_seam(A, gpu):
    import os
    import sys
    seam = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "adaptivetrainingsystem_amd",
                        "seams")
    sys.path.insert(0, seam)
    try:
        import cuda_opt_wrapper as cow
        from core.moe_cuda_wrapper import MoECUDAOps, MoEFFNLayer   # noqa: F401
    finally:
        sys.path.remove(seam)
    assert cow.TRANSFORMER_OPS_AVAILABLE
    F = torch.nn.functional

    def expect(m, x):
        gb = None if m.gate_proj.bias is None else m.gate_proj.bias.detach().float().cpu()
        ub = None if m.up_proj.bias is None else m.up_proj.bias.detach().float().cpu()
        gate = F.linear(x.float(), m.gate_proj.weight.detach().float().cpu(), gb)
        up = F.linear(x.float(), m.up_proj.weight.detach().float().cpu(), ub)
        return gate * F.silu(up)

    # float32, no biases, no autograd: one GEMM over the stacked weight with the activation in its epilogue
    m = cow.FusedSwiGLU(32, 48).to(gpu)
    x = torch.randn(2, 5, 32, generator=gen(23))
    with torch.no_grad():
        got = m(x.to(gpu)).cpu()
    assert got.shape == (2, 5, 48)
    assert rel_err(got, expect(m, x)) <= 1e-4
    # the stacked copy follows a write to a parameter
    with torch.no_grad():
        m.up_proj.weight.mul_(0.5)
        assert rel_err(m(x.to(gpu)).cpu(), expect(m, x)) <= 1e-4
    # bfloat16 at a prefill-sized and at a decode-sized row count (the second takes the K-sliced path)
    mb = cow.FusedSwiGLU(256, 512).to(gpu)
    for rows, seed in ((300, 24), (4, 25)):
        xb = torch.randn(rows, 256, generator=gen(seed)).bfloat16()
        with torch.no_grad():
            got = mb(xb.to(gpu)).float().cpu()
        wg, wu = (w.detach().bfloat16().float().cpu() for w in (mb.gate_proj.weight, mb.up_proj.weight))
        ref = F.linear(xb.float(), wg) * F.silu(F.linear(xb.float(), wu))
        assert rel_err(got, ref) <= 1e-2, rows
    # biases: the projections run as single-group GEMMs, the biases and the activation follow
    mbias = cow.FusedSwiGLU(32, 48, use_bias=True).to(gpu)
    with torch.no_grad():
        assert rel_err(mbias(x.to(gpu)).cpu(), expect(mbias, x)) <= 1e-4
    # autograd: gradients of the input, both weights and both biases against torch on the CPU
    xg = x.clone().to(gpu).requires_grad_(True)
    y = mbias(xg)
    dy = torch.randn(2, 5, 48, generator=gen(26))
    y.backward(dy.to(gpu))
    xc = x.clone().requires_grad_(True)
    ps = [p.detach().cpu().clone().requires_grad_(True) for p in (mbias.gate_proj.weight, mbias.gate_proj.bias,
                                                                  mbias.up_proj.weight, mbias.up_proj.bias)]
    yc = F.linear(xc, ps[0], ps[1]) * F.silu(F.linear(xc, ps[2], ps[3]))
    yc.backward(dy)
    assert rel_err(y.detach().cpu(), yc.detach()) <= 1e-4
    assert rel_err(xg.grad.cpu(), xc.grad) <= 1e-4
    for got_p, ref_p in zip((mbias.gate_proj.weight, mbias.gate_proj.bias, mbias.up_proj.weight, mbias.up_proj.bias), ps):
        assert rel_err(got_p.grad.cpu(), ref_p.grad) <= 1e-4
    with pytest.raises(A.AtsError):
        m(torch.randn(2, 31, device=gpu))


def test_decode_ffn_step_replays_in_a_hip_graph(A, gpu):
    """The K-sliced decode path allocates through torch and launches on the current stream, so a step can be
    captured: three replays with eager work and synchronisation in between, each equal to the eager result."""
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    ffn = A.DenseSwiGLU(LayerConfig(1024, 2048, 1, 1)).to(torch.bfloat16).to(gpu).eval()
    x = torch.randn(1, 8, 1024, generator=gen(71)).bfloat16().to(gpu)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):           # warm-up off the capturing stream: tables and caches get built
            for _ in range(2):
                ffn(x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y = ffn(x)
        for rep in range(3):
            x.copy_(torch.randn(1, 8, 1024, generator=gen(72 + rep)).bfloat16())
            ref = ffn(x)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, ref), rep


def test_mod_moe_block_replays_in_a_hip_graph(A, gpu):
    """The MoD + MoE block's inference path (score + copy pass, selection, gather, MoE layer whose combine adds
    onto the copy) launches on the current stream and never synchronises: captured once, three replays with
    eager work in between, each equal to the eager output and auxiliary loss."""
    from adaptivetrainingsystem_amd import workloads as W
    ov = {"batch": 4, "seq": 512, "hidden": 256, "intermediate": 128}
    w = W.make_moe_workload("c5_finegrained_mod", device=gpu, overrides=ov)
    block = W.build_layer(w, "fcfs")
    x = w.x
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                block(x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y, aux = block(x)
        for rep in range(3):
            x.copy_(torch.randn(x.shape, generator=gen(90 + rep)).to(x.dtype))
            ref, ref_aux = block(x)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, ref), rep
            assert torch.equal(aux, ref_aux), rep


def test_moe_decode_step_replays_in_a_hip_graph(A, gpu):
    """The inference path of the MoE layer never synchronises (the plan stays on the device), so a decoding
    step can be captured as well: replays equal the eager output and auxiliary loss."""
    from adaptivetrainingsystem_amd import workloads as W
    w = W.make_moe_workload("c3_decode", device=gpu, overrides={"hidden": 1024, "intermediate": 2048})
    layer = W.build_layer(w, "fcfs").eval()
    x = w.x
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                layer(x)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y, aux = layer(x)
        for rep in range(3):
            x.copy_(torch.randn(x.shape, generator=gen(80 + rep)).to(x.dtype))
            ref, ref_aux = layer(x)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, ref) and torch.equal(aux, ref_aux), rep


@pytest.mark.parametrize("counts,H,I,gather", [([900, 0, 1300, 1001], 256, 392, True), ([2100, 777], 512, 1024, False),
                                               ([800], 128, 136, True), ([1100, 1, 2303, 64, 0, 1216], 128, 200, False)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grouped_gateup_with_saved_preactivations(ops, gpu, counts, H, I, gather, dtype):
    """Training forward of the gate/up projection in one kernel: h has the bits of the inference kernel, the
    saved pre-activations have the bits of the plain product (same accumulation order), rows outside the
    groups are never written, and sizes below the prefill tile are declined (None), not computed."""
    print("case gateup save", counts, H, I, gather, dtype, flush=True)
    g = gen(61)
    E, n = len(counts), sum(counts)
    ws = [(torch.randn(2 * I, H, generator=g) * 0.05).to(dtype).to(gpu) for _ in range(E)]
    tab = ops.weight_pointer_table(ws)
    count = torch.tensor(counts, dtype=torch.int32)
    start = (torch.cumsum(count, 0) - count).to(torch.int32)
    rows = torch.randn(n, H, generator=g).to(dtype)
    pad = 7                                                # rows past the groups stay untouched
    if gather:
        k = 2
        T = n // k + 5
        src = torch.randn(T, H, generator=g).to(dtype)
        a_rows = torch.randint(0, T * k, (n,), generator=g).to(torch.int32)
        a, kw = src.to(gpu), dict(a_rows=a_rows.to(gpu), a_row_div=k)
        rows = src[(a_rows // k).long()]
    else:
        a, kw = rows.to(gpu), {}
    start, count = start.to(gpu), count.to(gpu)
    ks, kc = ops.wgrad_plan(count)
    both = ops.grouped_gateup_swiglu_save(a, tab, start, count, n + pad, n, H, I, t_col0=ks, **kw)
    assert both is not None
    gu, h, hT = both
    assert gu.shape == (n + pad, 2 * I) and h.shape == (n + pad, I) and gu.dtype == dtype and h.dtype == dtype
    # the transposed copy for the weight gradient: bfloat16 launches write it, with the bits of h and zero padding
    assert (hT is not None) == (dtype == torch.bfloat16)
    if hT is not None:
        want = ops.transpose_grouped_rows(h[:n], start, count, n)
        assert hT.shape == want.shape
        for e, c in enumerate(counts):
            lo, width = int(ks[e]), int(kc[e])
            assert width == max(64, (c + 63) // 64 * 64)
            assert same_bits(hT[:, lo:lo + width], want[:, lo:lo + width]), e
            assert torch.all(hT[:, lo + c:lo + width] == 0)
        plain = ops.grouped_gateup_swiglu_save(a, tab, start, count, n + pad, n, H, I, **kw)
        assert plain[2] is None and same_bits(plain[1][:n], h[:n]) and same_bits(plain[0][:n], gu[:n])
    h_inf = ops.grouped_gateup_swiglu(a, tab, start, count, n + pad, n, H, I, **kw)
    assert same_bits(h[:n], h_inf[:n])
    gu_plain = ops.grouped_gemm_nt(tab, H, 2 * I, start, count, n + pad, n, 2 * I, H, a=a, **kw)
    assert same_bits(gu[:n], gu_plain[:n])
    # against the oracle: float64 product per expert
    off = 0
    for e, c in enumerate(counts):
        if c:
            ref = rows[off:off + c].double() @ ws[e].cpu().double().T
            assert rel_err(gu[off:off + c], ref) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)
            ref_h = torch.nn.functional.silu(ref[:, :I]) * ref[:, I:]
            assert rel_err(h[off:off + c], ref_h) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)
        off += c
    # untouched tail: fill, run again into the same buffers through the C entry point, compare
    lib = __import__("adaptivetrainingsystem_amd._lib", fromlist=["load"]).load()
    gu.fill_(3.0)
    h.fill_(5.0)
    rc = lib.ats_grouped_gateup_swiglu_save(a.data_ptr(), a.shape[0], kw["a_rows"].data_ptr() if gather else None,
                                            kw.get("a_row_div", 1), tab.data_ptr(), h.data_ptr(), gu.data_ptr(),
                                            start.data_ptr(), count.data_ptr(), E, n, H, I,
                                            0 if dtype == torch.float32 else 1, None, 0, None, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.all(gu[n:] == 3.0) and torch.all(h[n:] == 5.0)
    assert same_bits(h[:n], h_inf[:n])
    # below the prefill tile the caller keeps the two-kernel route
    small = torch.tensor([40] * E, dtype=torch.int32, device=gpu)
    assert ops.grouped_gateup_swiglu_save(a, tab, start, small, n, 40 * E, H, I, **kw) is None


@pytest.mark.parametrize("counts,K,N", [([900, 0, 300, 1001], 256, 392), ([2100, 777], 1024, 512), ([300], 128, 136),
                                        ([1024, 1, 1279, 64, 0, 193], 192, 200), ([513], 64, 8), ([700, 700], 448, 1000)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_grouped_gemm_against_k_major_weights(ops, gpu, counts, K, N, out_dtype):
    """out = A . B with B stored [K, N] (the forward's weights in a data gradient): the bits of the NT product
    against the transposed copy, agreement with float64, rows outside the groups untouched, gathered A rows,
    and the sizes it declines."""
    print("case gemm nn", counts, K, N, out_dtype, flush=True)
    g = gen(167)
    E, n = len(counts), sum(counts)
    w = [(torch.randn(K, N, generator=g) * 0.05).bfloat16().to(gpu) for _ in range(E)]
    wT = [x.t().contiguous() for x in w]
    tab, tabT = ops.weight_pointer_table(w), ops.weight_pointer_table(wT)
    count = torch.tensor(counts, dtype=torch.int32)
    start = (torch.cumsum(count, 0) - count).to(torch.int32).to(gpu)
    count = count.to(gpu)
    a = torch.randn(n + 3, K, generator=g).bfloat16().to(gpu)
    assert ops.grouped_gemm_nn_supported(E, n, N, K, N, torch.bfloat16)
    out = ops.grouped_gemm_nn(tab, N, start, count, n + 3, n, N, K, a, out_dtype=out_dtype)
    ref = ops.grouped_gemm_nt(tabT, K, N, start, count, n + 3, n, N, K, a=a, out_dtype=out_dtype)
    assert out.dtype == out_dtype and same_bits(out[:n], ref[:n])
    off = 0
    for e, c in enumerate(counts):
        if c:
            r64 = a[off:off + c].cpu().double() @ w[e].cpu().double()
            assert rel_err(out[off:off + c], r64) <= BF16_TOL
        off += c
    # gathered rows of A (row m of the product reads a[src[m] // 2])
    src = torch.randint(0, 2 * (n + 3), (n,), generator=g).to(torch.int32).to(gpu)
    got = ops.grouped_gemm_nn(tab, N, start, count, n, n, N, K, a, a_rows=src, a_row_div=2, out_dtype=out_dtype)
    want = ops.grouped_gemm_nn(tab, N, start, count, n, n, N, K, a[(src // 2).long()].contiguous(), out_dtype=out_dtype)
    assert same_bits(got, want)
    # rows beyond the groups are not written
    lib = __import__("adaptivetrainingsystem_amd._lib", fromlist=["load"]).load()
    buf = torch.full((n + 3, N), 7.0, dtype=out_dtype, device=gpu)
    rc = lib.ats_grouped_gemm_nn(a.data_ptr(), K, n + 3, None, 1, tab.data_ptr(), N, buf.data_ptr(), N, start.data_ptr(),
                                 count.data_ptr(), E, n, N, K, 1, 0 if out_dtype == torch.float32 else 1, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.all(buf[n:] == 7.0) and same_bits(buf[:n], ref[:n])
    # declined: decode-sized groups, float32 operands, K not a multiple of 64
    assert not ops.grouped_gemm_nn_supported(E, 40 * E, N, K, N, torch.bfloat16)
    assert not ops.grouped_gemm_nn_supported(E, n, N, K, N, torch.float32)
    assert not ops.grouped_gemm_nn_supported(E, n, N, K + 8, N, torch.bfloat16)
    assert lib.ats_grouped_gemm_nn(a.data_ptr(), K, n + 3, None, 1, tab.data_ptr(), N, buf.data_ptr(), N, start.data_ptr(),
                                   count.data_ptr(), E, 40 * E, N, K, 1, 1, None) == -2


@pytest.mark.parametrize("counts,H,I", [([900, 0, 300, 1001], 256, 392), ([2100, 777], 512, 1024), ([300], 128, 136),
                                        ([1024, 1, 1279, 64, 0, 193], 128, 200)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_grouped_down_dgrad_with_swiglu_gradient(ops, gpu, counts, H, I, dtype):
    """Training backward in one kernel: dgu has the bits of the plain product dh = dy . Wd followed by the
    elementwise gradient of silu(g) * u, agrees with the float64 formula, leaves rows outside the groups
    alone, and declines sizes below the prefill tile."""
    print("case dgrad dsilu", counts, H, I, dtype, flush=True)
    g = gen(67)
    E, n = len(counts), sum(counts)
    wdT = [(torch.randn(I, H, generator=g) * 0.05).to(dtype).to(gpu) for _ in range(E)]     # Wd^T per expert
    tab = ops.weight_pointer_table(wdT)
    count = torch.tensor(counts, dtype=torch.int32)
    start = (torch.cumsum(count, 0) - count).to(torch.int32).to(gpu)
    count = count.to(gpu)
    pad = 5
    dy = torch.randn(n + pad, H, generator=g).to(dtype).to(gpu)
    gu = torch.randn(n + pad, 2 * I, generator=g).to(dtype).to(gpu)
    ks, kc = ops.wgrad_plan(count)
    pair = ops.grouped_down_dgrad_dsilu(dy, tab, gu, start, count, n, H, I, t_col0=ks)
    assert pair is not None
    dgu, dguT = pair
    assert dgu.shape == gu.shape and dgu.dtype == dtype
    assert (dguT is not None) == (dtype == torch.bfloat16)
    if dguT is not None:
        want = ops.transpose_grouped_rows(dgu[:n], start, count, n)
        assert dguT.shape == want.shape
        for e, c in enumerate(counts):
            lo, width = int(ks[e]), int(kc[e])
            assert same_bits(dguT[:, lo:lo + width], want[:, lo:lo + width]), e
            assert torch.all(dguT[:, lo + c:lo + width] == 0)
        plain = ops.grouped_down_dgrad_dsilu(dy, tab, gu, start, count, n, H, I)
        assert plain[1] is None and same_bits(plain[0][:n], dgu[:n])
    dh = ops.grouped_gemm_nt(tab, H, I, start, count, n + pad, n, I, H, a=dy)
    two = torch.empty_like(gu)
    ops.silu_mul_bwd(gu[:n, :I], gu[:n, I:], dh[:n], da=two[:n, :I], db=two[:n, I:])
    assert same_bits(dgu[:n], two[:n])
    off = 0
    for e, c in enumerate(counts):
        if c:
            dh64 = dy[off:off + c].cpu().double() @ wdT[e].cpu().double().T
            if dtype == torch.bfloat16:
                dh64 = dh64.bfloat16().double()                 # dh is rounded before the gradient, as when stored
            g64, u64 = gu[off:off + c, :I].cpu().double(), gu[off:off + c, I:].cpu().double()
            s64 = torch.sigmoid(g64)
            ref = torch.cat([dh64 * u64 * (s64 + g64 * s64 * (1 - s64)), dh64 * g64 * s64], dim=1)
            assert rel_err(dgu[off:off + c], ref) <= (F32_TOL if dtype == torch.float32 else BF16_TOL)
        off += c
    # the forward's own weights ([H, I] per expert) instead of the transposed copy: bfloat16, H a multiple of 64
    wd = [x.t().contiguous() for x in wdT]
    nn = ops.grouped_down_dgrad_dsilu(dy, ops.weight_pointer_table(wd), gu, start, count, n, H, I, t_col0=ks,
                                      transposed_weights=False)
    assert (nn is not None) == (dtype == torch.bfloat16 and H % 64 == 0)
    if nn is not None:
        assert same_bits(nn[0][:n], dgu[:n])
        for e in range(E):
            lo, width = int(ks[e]), int(kc[e])
            assert same_bits(nn[1][:, lo:lo + width], dguT[:, lo:lo + width]), e
    lib = __import__("adaptivetrainingsystem_amd._lib", fromlist=["load"]).load()
    dgu.fill_(3.0)
    rc = lib.ats_grouped_down_dgrad_dsilu(dy.data_ptr(), tab.data_ptr(), gu.data_ptr(), dgu.data_ptr(), start.data_ptr(),
                                          count.data_ptr(), E, n, H, I, 0 if dtype == torch.float32 else 1,
                                          None, 0, None, None)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.all(dgu[n:] == 3.0) and same_bits(dgu[:n], two[:n])
    small = torch.tensor([40] * E, dtype=torch.int32, device=gpu)
    assert ops.grouped_down_dgrad_dsilu(dy, tab, gu, start, small, 40 * E, H, I) is None


@pytest.mark.parametrize("T,H,dtype", [(300, 2048, torch.bfloat16), (17, 33, torch.bfloat16), (64, 516, torch.float32),
                                       (5, 7, torch.float32)])
def test_row_dot_with_copy(ops, gpu, T, H, dtype):
    """The MoD score pass that also writes the rows it reads: the same scores bit for bit, an exact copy."""
    x = torch.randn(T, H, generator=gen(91)).to(dtype).to(gpu)
    w = torch.randn(H, generator=gen(92)).to(dtype).to(gpu)
    plain = ops.row_dot(x, w)
    score, prob, copy = ops.row_dot(x, w, temperature=0.7, want_prob=True, want_copy=True)
    assert same_bits(score, plain)
    assert copy.data_ptr() != x.data_ptr() and torch.equal(copy, x)
    assert rel_err(prob, torch.sigmoid(plain.cpu().double() / 0.7)) <= 1e-6
    score2, copy2 = ops.row_dot(x, w, want_copy=True)
    assert same_bits(score2, plain) and torch.equal(copy2, x)
    lib = __import__("adaptivetrainingsystem_amd._lib", fromlist=["load"]).load()
    assert lib.ats_row_dot_copy(x.data_ptr(), w.data_ptr(), None, score.data_ptr(), None, 1.0, x.data_ptr(), T, H,
                                0 if dtype == torch.float32 else 1, None) != 0       # the copy may not alias x


@pytest.mark.parametrize("T,k,H,N,ydt,odt", [(300, 6, 2048, 1000, torch.bfloat16, torch.bfloat16),
                                             (4200, 2, 2048, 5000, torch.bfloat16, torch.bfloat16),
                                             (64, 8, 520, 64, torch.float32, torch.float32),
                                             (129, 3, 64, 400, torch.float32, torch.bfloat16)])
def test_combine_scatter_add_equals_combine_then_scatter_add(ops, gpu, T, k, H, N, ydt, odt):
    """The combine that adds its token-major result onto rows of a larger tensor: the bits of combine followed
    by scatter_add_rows, rows with a negative destination skipped, other rows of the target untouched; sizes
    outside the vector kernel are declined."""
    g = gen(95)
    rows = T * k
    y = torch.randn(rows, H, generator=g).to(ydt).to(gpu)
    row_of = torch.randperm(rows, generator=g).int()
    row_of[torch.rand(rows, generator=g) < 0.1] = -1                   # dropped choices
    w = torch.rand(T, k, generator=g).to(gpu)
    dest = torch.randperm(N, generator=g)[:T].int()
    dest[::17] = -1
    base = torch.randn(N, H, generator=g).to(odt).to(gpu)
    row_of, dest = row_of.to(gpu), dest.to(gpu)
    two = base.clone()
    ops.scatter_add_rows(two, dest, ops.combine(y, row_of, w, T, k, out_dtype=odt))
    one = base.clone()
    assert ops.combine_scatter_add(y, row_of, w, T, k, one, dest)
    assert same_bits(one, two)
    untouched = torch.ones(N, dtype=torch.bool)
    untouched[dest[dest >= 0].long().cpu()] = False
    assert torch.equal(one[untouched.to(gpu)], base[untouched.to(gpu)])
    odd = torch.zeros(N, 260, dtype=odt, device=gpu)
    assert not ops.combine_scatter_add(torch.zeros(rows, 260, dtype=ydt, device=gpu), row_of, w, T, k, odd, dest)


@pytest.mark.parametrize("n,kth", [(1, 1), (150, 75), (5000, 1), (5000, 5000), (16384, 8000), (40000, 1), (40000, 40000),
                                   (100003, 50002), (300000, 299999)])
def test_kth_value_mask_both_selects(ops, gpu, n, kth):
    """mask = values >= the kth smallest value (model.py:984-990), by the single-workgroup radix select (small n,
    or a 16-byte workspace) and by the one-launch-per-digit select over many workgroups (from 16384 values on):
    against torch.kthvalue on the CPU, with heavy ties, negative values, signed zeros and infinities; the count of
    ones is the mask's sum; both selects agree."""
    g = gen(400 + n % 97)
    v = torch.randn(n, generator=g)
    v[torch.rand(n, generator=g) < 0.3] = 0.25                 # a third of the values tie
    if n >= 150:
        v[:4] = torch.tensor([float("inf"), float("-inf"), 0.0, -0.0])
    thr = torch.kthvalue(v, kth).values
    ref = (v >= thr).float()
    mask, count = ops.kth_value_mask(v.to(gpu), kth, return_count=True)
    assert torch.equal(mask.cpu(), ref)
    assert count.item() == int(ref.sum().item())
    # the single-workgroup select through the C ABI (a 16-byte workspace keeps it at any size)
    lib = __import__("adaptivetrainingsystem_amd._lib", fromlist=["load"]).load()
    vg = v.to(gpu)
    m2 = torch.empty_like(vg)
    ws = torch.empty(2, dtype=torch.int64, device=gpu)
    assert lib.ats_kth_value_mask(vg.data_ptr(), n, kth, m2.data_ptr(), ws.data_ptr(), 16, None) == 0
    torch.cuda.synchronize()
    assert torch.equal(m2.cpu(), ref) and ws[1].item() == int(ref.sum().item())
    assert int(lib.ats_kth_value_workspace(n)) == (16 if n < 16384 else 16 + 4096)


# ------------------------------------------------------------------ float16 activations
def test_float16_activations_run_through_the_float32_kernels(A, gpu):
    """float16 is served as the reference's fused wrappers serve every dtype (cuda_opt_wrapper.py:92, 117, 153, 217):
    up-cast, float32 kernels, one rounding back.  Norm and RoPE also train that way; the layers with weight
    matrices take float16 for inference and refuse to train in it."""
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    g = gen(91)
    x = torch.randn(3, 17, 256, generator=g).half()
    norm = A.RMSNorm(256).to(gpu)
    with torch.no_grad():
        norm.weight.copy_(torch.randn(256, generator=g) * 0.1 + 1.0)
    y = norm(x.to(gpu))
    ref = O.rmsnorm(x.float(), norm.weight.detach().cpu(), 1e-6)
    assert y.dtype == torch.float16 and rel_err(y, ref) <= 2 ** -10
    xg = x.to(gpu).requires_grad_()
    norm(xg).float().sum().backward()
    xr = x.float().requires_grad_()
    O.rmsnorm(xr, norm.weight.detach().cpu(), 1e-6).sum().backward()
    assert xg.grad.dtype == torch.float16 and rel_err(xg.grad, xr.grad) <= 2e-3
    fused = A.FusedRMSNorm(256).to(gpu).half()
    assert fused(x.to(gpu)).dtype == torch.float16
    q = torch.randn(2, 4, 33, 64, generator=g).half()
    k = torch.randn(2, 2, 33, 64, generator=g).half()
    cos, sin = A.RotaryEmbedding(64, max_seq_len=64)(33, gpu)
    gq, gk = A.apply_rotary_pos_emb(q.to(gpu), k.to(gpu), cos, sin)
    rq, rk = O.rope_apply(q.float(), k.float(), cos.cpu(), sin.cpu())
    assert gq.dtype == torch.float16 and rel_err(gq, rq) <= 2 ** -10 and rel_err(gk, rk) <= 2 ** -10
    fq, fk = A.FusedRoPE(64, max_seq_len=64)(q.to(gpu), k.to(gpu), 3)
    assert fq.dtype == torch.float16 and fk.shape == k.shape
    # MoE layer, dense FFN and attention: float16 inference against the oracle on float32 copies
    cfg = LayerConfig(128, 256, 4, 2, 1.25, num_heads=4, num_kv_heads=2, seq_length=64, moe_capacity_mode="fcfs")
    torch.manual_seed(3)
    moe = A.MoEFFNLayer(cfg).to(gpu).half().eval()
    xm = torch.randn(2, 24, 128, generator=g).half()
    with torch.no_grad():
        out, aux = moe(xm.to(gpu))
    p = moe.last_plan
    refm = O.moe_forward_capacity(xm.float(), moe.gate.weight.detach().float().cpu(),
                                  [e.gate_up_proj.weight.detach().float().cpu() for e in moe.experts],
                                  [e.down_proj.weight.detach().float().cpu() for e in moe.experts], k=2,
                                  capacity_factor=1.25, logits_override=p["logits"].cpu())
    assert out.dtype == torch.float16 and rel_err(out, refm["out"].reshape(out.shape)) <= 2e-3
    ffn = A.DenseSwiGLU(cfg).to(gpu).half().eval()
    with torch.no_grad():
        yf = ffn(xm.to(gpu))
    assert yf.dtype == torch.float16
    assert rel_err(yf, O.swiglu_expert(xm.float(), ffn.gate_up_proj.weight.detach().float().cpu(),
                                       ffn.down_proj.weight.detach().float().cpu())) <= 2e-3
    att = A.GroupedQueryAttention(cfg).to(gpu).half().eval()
    with torch.no_grad():
        ya, (kc, vc) = att(xm.to(gpu), use_cache=True)
    w = [getattr(att, n).weight.detach().float().cpu() for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
    assert ya.dtype == kc.dtype == vc.dtype == torch.float16
    assert rel_err(ya, O.gqa_forward(xm.float(), *w, 4, 2)) <= 5e-3
    moe.train()
    with pytest.raises(A.AtsError):
        moe(xm.to(gpu).requires_grad_())
    from adaptivetrainingsystem_amd.seams import cuda_opt_wrapper as cow
    sw = cow.FusedSwiGLU(128, 192).to(gpu).half().eval()
    with torch.no_grad():
        ys = sw(xm.to(gpu))
    gate = xm.float() @ sw.gate_proj.weight.detach().float().cpu().t()
    up = xm.float() @ sw.up_proj.weight.detach().float().cpu().t()
    assert ys.dtype == torch.float16 and rel_err(ys, gate * torch.nn.functional.silu(up)) <= 2e-3
    with pytest.raises(A.AtsError):
        sw(xm.to(gpu).requires_grad_())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_transposed_zero_empty_groups(ops, gpu, dtype):
    """The 64 columns of every expert without rows are cleared in a transposed [C, ld] matrix; nothing else is touched."""
    lib = __import__("adaptivetrainingsystem_amd._lib", fromlist=["load"]).load()
    counts = torch.tensor([5, 0, 130, 0, 0, 64], dtype=torch.int32, device=gpu)
    ks, kc = ops.wgrad_plan(counts)
    E, C = counts.numel(), 37
    ld = ops.wgrad_padded_rows(int(counts.sum()), E)
    buf = torch.full((C, ld), 7.0, dtype=dtype, device=gpu)
    rc = lib.ats_transposed_zero_empty_groups(buf.data_ptr(), ld, C, counts.data_ptr(), ks.data_ptr(), E,
                                              0 if dtype == torch.float32 else 1, None)
    assert rc == 0
    torch.cuda.synchronize()
    want = torch.full((C, ld), 7.0, dtype=dtype)
    for e in range(E):
        if int(counts[e]) == 0:
            assert int(kc[e]) == 64
            want[:, int(ks[e]):int(ks[e]) + 64] = 0
    assert torch.equal(buf.cpu(), want)
    assert lib.ats_transposed_zero_empty_groups(buf.data_ptr(), ld + 1, C, counts.data_ptr(), ks.data_ptr(), E, 1, None) != 0
