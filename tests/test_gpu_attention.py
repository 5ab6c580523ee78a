"""Parity of the causal grouped-query attention kernel and module against the CPU oracle (restatement of
the reference's _standard_attention and GroupedQueryAttention.forward), through the C ABI.  bf16 bar:
2e-2 of the oracle's max-abs."""
import pytest
import torch

from oracle import sparse_layer_oracle as O

pytestmark = pytest.mark.gpu
BF16_TOL = 2e-2


def rel_err(got, ref) -> float:
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.fixture(scope="module")
def ops(gpu):
    from adaptivetrainingsystem_amd import _lib, ops as _ops
    _lib.load()
    return _ops


@pytest.mark.parametrize("B,Hq,Hkv,L,D", [(1, 2, 1, 64, 128), (2, 4, 2, 200, 128), (1, 8, 2, 513, 64), (1, 1, 1, 1, 128),
                                          (2, 3, 3, 129, 64), (1, 4, 1, 1024, 128), (1, 2, 2, 31, 64),
                                          (1, 2, 1, 4100, 64), (1, 1, 1, 4300, 128)])      # 8-wave blocks from 4096 on
def test_causal_attention(ops, gpu, B, Hq, Hkv, L, D):
    print("case attention", B, Hq, Hkv, L, D, flush=True)
    g = gen(91)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    rep = Hq // Hkv
    ref = O.attention_standard(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1), D ** -0.5)
    out, lse = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), return_lse=True)
    assert out.shape == (B, L, Hq * D) and out.dtype == torch.bfloat16
    assert rel_err(out, ref) <= BF16_TOL
    s = torch.matmul(q.float(), k.repeat_interleave(rep, dim=1).float().transpose(-2, -1)) * D ** -0.5
    s = s.masked_fill(torch.triu(torch.ones(L, L, dtype=torch.bool), diagonal=1), float("-inf"))
    assert rel_err(lse, torch.logsumexp(s, -1)) <= 1e-4
    # v given as a strided view of a fused projection output [B, L, Hkv, D]
    v_view = v.transpose(1, 2).contiguous().to(gpu).transpose(1, 2)
    out2 = ops.causal_attention(q.to(gpu), k.to(gpu), v_view)
    assert torch.equal(out2, out)


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D", [(2, 4, 2, 1, 200, 128), (1, 2, 1, 1, 1, 64), (1, 4, 4, 70, 300, 64),
                                             (3, 8, 2, 1, 513, 128), (2, 32, 8, 3, 100, 64), (1, 12, 2, 40, 77, 128),
                                             (1, 16, 2, 127, 127, 64), (2, 6, 3, 33, 1000, 128),
                                             (2, 8, 2, 129, 130, 128), (1, 2, 2, 256, 1024, 128), (1, 4, 1, 5, 64, 128)])
def test_causal_attention_with_cached_keys(ops, gpu, B, Hq, Hkv, L, Lk, D):
    """Lk - L cached keys in front of the queries: query i sees keys 0 .. i + Lk - L."""
    print("case cached attention", B, Hq, Hkv, L, Lk, D, flush=True)
    g = gen(94)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    rep = Hq // Hkv
    ref = O.attention_standard(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1), D ** -0.5)
    out, lse = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), return_lse=True)
    assert out.shape == (B, L, Hq * D)
    assert rel_err(out, ref) <= BF16_TOL
    s = torch.matmul(q.float(), k.repeat_interleave(rep, dim=1).float().transpose(-2, -1)) * D ** -0.5
    s = s.masked_fill(torch.triu(torch.ones(L, Lk, dtype=torch.bool), diagonal=1 + Lk - L), float("-inf"))
    assert rel_err(lse, torch.logsumexp(s, -1)) <= 1e-4


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D", [(1, 32, 8, 1, 2048, 128), (2, 8, 2, 1, 4097, 64), (1, 4, 4, 1, 300, 128),
                                             (3, 8, 2, 5, 1000, 128), (1, 16, 2, 16, 515, 64), (5, 2, 1, 64, 700, 128)])
def test_decode_attention_over_key_ranges(ops, gpu, B, Hq, Hkv, L, Lk, D):
    """Few query rows against many keys: the keys are cut into ranges that run side by side and are merged.
    Same result as the single pass (to float32 rounding of the merge), the oracle's values, the log-sum-exp,
    and the padding bias carried through the ranges."""
    from adaptivetrainingsystem_amd import _lib
    print("case key ranges", B, Hq, Hkv, L, Lk, D, flush=True)
    assert _lib.load().ats_attention_fwd_workspace(B, Hq, Hkv, L, Lk, D) > 0
    g = gen(140)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    rep = Hq // Hkv
    for mask in (None, _padding_mask(B, Lk, 141)):
        if mask is not None:
            mask[:, :Lk - L + 1] = 1
            mask[:, 70:130] = 0            # a stretch of padded keys inside the cache
        bias = None if mask is None else ((1.0 - mask) * -1e4).to(gpu)
        ref = O.attention_standard(q, k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1), D ** -0.5, mask)
        out, lse = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), return_lse=True, key_bias=bias)
        one, lse1 = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), return_lse=True, key_bias=bias, split_keys=False)
        assert rel_err(out, ref) <= BF16_TOL
        assert rel_err(out, one) <= 1e-2 and rel_err(lse, lse1) <= 1e-5


def test_cached_attention_equals_tail_of_full_call(ops, gpu):
    """Size-independent property at a long length: the last L rows of a full call, bit for bit per row tile
    alignment aside -- compared at the bf16 bar since tiles start at different keys."""
    g = gen(95)
    B, Hq, Hkv, Lk, D, L = 1, 8, 2, 4096, 128, 1024
    q = torch.randn(B, Hq, Lk, D, generator=g).bfloat16().to(gpu)
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16().to(gpu)
    full = ops.causal_attention(q, k, v)
    tail = ops.causal_attention(q[:, :, Lk - L:], k, v)
    assert rel_err(tail, full[:, Lk - L:]) <= 1e-6      # same keys, same tile walk: identical arithmetic
    with pytest.raises(Exception):
        ops.causal_attention(q, k[:, :, :100], v[:, :, :100])          # fewer keys than queries


def test_attention_is_causal(ops, gpu):
    """Changing keys / values at later positions must not change earlier outputs (bit for bit)."""
    g = gen(92)
    B, Hq, Hkv, L, D = 1, 4, 2, 300, 128
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16().to(gpu)
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16().to(gpu)
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16().to(gpu)
    base = ops.causal_attention(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[:, :, 170:] = 5.0
    v2[:, :, 170:] = -3.0
    out = ops.causal_attention(q, k2, v2)
    assert torch.equal(out[:, :170], base[:, :170]) and not torch.equal(out[:, 170:], base[:, 170:])


@pytest.mark.parametrize("hidden,nh,nkv,B,L", [(512, 4, 2, 2, 77), (1024, 8, 8, 1, 256), (256, 4, 1, 3, 130)])
def test_gqa_module(gpu, hidden, nh, nkv, B, L):
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    print("case gqa module", hidden, nh, nkv, B, L, flush=True)
    torch.manual_seed(13)
    cfg = LayerConfig(hidden, 4 * hidden, 1, 1, num_heads=nh, num_kv_heads=nkv, seq_length=512)
    att = A.GroupedQueryAttention(cfg)
    with torch.no_grad():
        for p in att.parameters():
            p.mul_(20.0)                       # scores of order one, so the softmax is not flat
    att = att.to(torch.bfloat16).to(gpu).eval()
    x = torch.randn(B, L, hidden, generator=gen(93)).bfloat16()
    ref = O.gqa_forward(x, att.q_proj.weight.detach().cpu(), att.k_proj.weight.detach().cpu(),
                        att.v_proj.weight.detach().cpu(), att.o_proj.weight.detach().cpu(), nh, nkv)
    with torch.no_grad():
        out = att(x.to(gpu))
    assert out.shape == x.shape and rel_err(out, ref) <= BF16_TOL
    assert set(att.state_dict()) == {f"{n}.weight" for n in ("q_proj", "k_proj", "v_proj", "o_proj")}
    # the stacked q/k/v weight of the inference path follows in-place updates and replaced parameters
    with torch.no_grad():
        att.k_proj.weight.mul_(0.5)
        w_k = att.k_proj.weight.detach().cpu()
        ref2 = O.gqa_forward(x, att.q_proj.weight.detach().cpu(), w_k, att.v_proj.weight.detach().cpu(),
                             att.o_proj.weight.detach().cpu(), nh, nkv)
        out2 = att(x.to(gpu))
        assert rel_err(out2, ref2) <= BF16_TOL and not torch.equal(out2, out)
        att.k_proj.weight = torch.nn.Parameter(att.k_proj.weight.detach() * 2.0)
        assert torch.equal(att(x.to(gpu)), out)
        att.k_proj.weight.data.mul_(0.5)          # a write the version counter does not see
        att.reset_cached_weights()
        assert torch.equal(att(x.to(gpu)), out2)
        att.k_proj.weight.data.mul_(2.0)
        att.reset_cached_weights()
    # prefill with use_cache, then two single-token steps fed from the cache (model.py:700-708)
    w = [getattr(att, n).weight.detach().cpu() for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
    with torch.no_grad():
        out_c, cache = att(x.to(gpu), use_cache=True)
    ref_c, ref_cache = O.gqa_forward(x, *w, nh, nkv, use_cache=True)
    assert torch.equal(out_c, out) and rel_err(cache[0], ref_cache[0]) <= BF16_TOL
    assert rel_err(cache[1], ref_cache[1]) <= BF16_TOL
    for step in range(2):
        x1 = torch.randn(B, 1, hidden, generator=gen(96 + step)).bfloat16()
        with torch.no_grad():
            o1, cache = att(x1.to(gpu), past_key_value=cache, use_cache=True)
        r1, ref_cache = O.gqa_forward(x1, *w, nh, nkv, past_key_value=ref_cache, use_cache=True)
        assert cache[0].shape == (B, nkv, L + 1 + step, hidden // nh)
        assert rel_err(o1, r1) <= BF16_TOL


# --------------------------------------------------------------------------- backward
GRAD_TOL = 2e-2      # bf16 bar on gradients, relative to the oracle gradient's max-abs


def _oracle_attention_grads(q, k, v, dout, rep):
    """Autograd through the oracle forward on float32 leaves holding the same bf16 values."""
    q32, k32, v32 = (t.float().requires_grad_() for t in (q, k, v))
    D = q.shape[-1]
    out = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5)
    out.backward(dout.float())
    return q32.grad, k32.grad, v32.grad


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D", [(1, 2, 1, 64, 64, 128), (2, 4, 2, 200, 200, 128), (1, 8, 2, 300, 300, 64),
                                             (1, 1, 1, 1, 1, 128), (2, 3, 3, 129, 129, 64), (1, 4, 1, 520, 520, 128),
                                             (1, 4, 2, 70, 300, 64), (2, 2, 1, 1, 130, 128), (1, 2, 2, 31, 31, 64)])
def test_causal_attention_backward(ops, gpu, B, Hq, Hkv, L, Lk, D):
    print("case attention backward", B, Hq, Hkv, L, Lk, D, flush=True)
    g = gen(97)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    rq, rk, rv = _oracle_attention_grads(q, k, v, dout, Hq // Hkv)
    out, lse = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), return_lse=True)
    dq, dk, dv = ops.causal_attention_bwd(q.to(gpu), k.to(gpu), v.to(gpu), out, lse, dout.to(gpu))
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    assert rel_err(dv, rv) <= GRAD_TOL
    assert rel_err(dq, rq) <= GRAD_TOL
    assert rel_err(dk, rk) <= GRAD_TOL


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D", [(2, 4, 2, 200, 200, 128), (1, 8, 2, 300, 300, 64), (1, 4, 2, 70, 300, 64),
                                             (1, 2, 2, 31, 31, 64)])
def test_causal_attention_backward_given_delta(ops, gpu, B, Hq, Hkv, L, Lk, D):
    """ats_attention_delta + ats_attention_bwd (delta computed by its own kernel and passed in) against the oracle
    and against the entry point that forms delta inside the dQ kernel (what ops.causal_attention_bwd calls)."""
    from adaptivetrainingsystem_amd import _lib
    print("case attention backward, given delta", B, Hq, Hkv, L, Lk, D, flush=True)
    g = gen(197)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    rq, rk, rv = _oracle_attention_grads(q, k, v, dout, Hq // Hkv)
    qg, kg, vg, dg = q.to(gpu), k.to(gpu), v.to(gpu), dout.to(gpu)
    out, lse = ops.causal_attention(qg, kg, vg, return_lse=True)
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    delta = torch.empty(B, Hq, L, dtype=torch.float32, device=gpu)
    assert lib.ats_attention_delta(out.data_ptr(), dg.data_ptr(), delta.data_ptr(), B, Hq, L, D, stream) == 0
    ref_delta = (out.float() * dg.float()).view(B, L, Hq, D).sum(-1).permute(0, 2, 1)
    assert rel_err(delta, ref_delta) <= 1e-5
    dq, dk, dv = torch.empty_like(qg), torch.empty_like(kg), torch.empty_like(vg)
    assert lib.ats_attention_bwd(qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), dg.data_ptr(), lse.data_ptr(),
                                 delta.data_ptr(), None, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), B, Hq, Hkv, L, Lk, D,
                                 float(D ** -0.5), stream) == 0
    for got, ref in ((dq, rq), (dk, rk), (dv, rv)):
        assert rel_err(got, ref) <= GRAD_TOL
    # the fused entry point leaves the same delta behind (summed in another order) and the same gradients
    delta2 = torch.full((B, Hq, L), float("nan"), dtype=torch.float32, device=gpu)
    dq2, dk2, dv2 = torch.empty_like(qg), torch.empty_like(kg), torch.empty_like(vg)
    assert lib.ats_attention_bwd_out(qg.data_ptr(), kg.data_ptr(), vg.data_ptr(), out.data_ptr(), dg.data_ptr(),
                                     lse.data_ptr(), delta2.data_ptr(), None, None, 0, 0, 0.0, 0, dq2.data_ptr(),
                                     dk2.data_ptr(), dv2.data_ptr(), B, Hq, Hkv, L, Lk, D, float(D ** -0.5), stream) == 0
    assert rel_err(delta2, ref_delta) <= 1e-5
    for got, ref in ((dq2, dq), (dk2, dk), (dv2, dv)):
        assert rel_err(got, ref) <= 1e-2


def test_attention_function_autograd(gpu):
    """The autograd Function: strided q/k/v views in, gradient accumulation through views out."""
    from adaptivetrainingsystem_amd.autograd import AttentionFunction
    g = gen(98)
    B, Hq, Hkv, L, D = 2, 4, 2, 150, 64
    base = [torch.randn(B, L, h, D, generator=g).bfloat16() for h in (Hq, Hkv, Hkv)]
    leaves = [t.to(gpu).requires_grad_() for t in base]
    q, k, v = (t.transpose(1, 2) for t in leaves)
    out = AttentionFunction.apply(q, k, v, D ** -0.5)
    w = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    (out.float() * w.to(gpu).float()).sum().backward()
    rq, rk, rv = _oracle_attention_grads(*(t.transpose(1, 2) for t in base), w, Hq // Hkv)
    for got, ref in zip(leaves, (rq, rk, rv)):
        assert rel_err(got.grad.transpose(1, 2), ref) <= GRAD_TOL


@pytest.mark.parametrize("T,K,N", [(300, 256, 192), (64, 128, 128), (1, 64, 320), (1000, 512, 64)])
def test_linear_function_grads(gpu, T, K, N):
    from adaptivetrainingsystem_amd.autograd import LinearFunction
    print("case linear function", T, K, N, flush=True)
    g = gen(99)
    x = torch.randn(T, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.1).bfloat16()
    dy = torch.randn(T, N, generator=g).bfloat16()
    xg, wg = x.to(gpu).requires_grad_(), w.to(gpu).requires_grad_()
    y = LinearFunction.apply(xg, wg)
    y.backward(dy.to(gpu))
    x32, w32 = x.float().requires_grad_(), w.float().requires_grad_()
    y32 = x32 @ w32.T
    y32.backward(dy.float())
    assert rel_err(y, y32) <= BF16_TOL
    assert rel_err(xg.grad, x32.grad) <= GRAD_TOL and rel_err(wg.grad, w32.grad) <= GRAD_TOL


@pytest.mark.parametrize("hidden,nh,nkv,B,L", [(512, 4, 2, 2, 77), (256, 4, 1, 1, 200)])
def test_gqa_module_backward(gpu, hidden, nh, nkv, B, L):
    """Input and parameter gradients of the whole attention sub-layer against autograd over the oracle forward."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    print("case gqa module backward", hidden, nh, nkv, B, L, flush=True)
    torch.manual_seed(14)
    cfg = LayerConfig(hidden, 4 * hidden, 1, 1, num_heads=nh, num_kv_heads=nkv, seq_length=512)
    att = A.GroupedQueryAttention(cfg)
    with torch.no_grad():
        for p in att.parameters():
            p.mul_(20.0)
    att = att.to(torch.bfloat16).to(gpu).train()
    x = torch.randn(B, L, hidden, generator=gen(100)).bfloat16()
    dy = torch.randn(B, L, hidden, generator=gen(101)).bfloat16()
    xg = x.to(gpu).requires_grad_()
    out = att(xg)
    out.backward(dy.to(gpu))
    names = ("q_proj", "k_proj", "v_proj", "o_proj")
    w32 = [getattr(att, n).weight.detach().float().cpu().requires_grad_() for n in names]
    x32 = x.float().requires_grad_()
    ref = O.gqa_forward(x32, *w32, nh, nkv)
    ref.backward(dy.float())
    assert rel_err(out, ref) <= BF16_TOL
    assert rel_err(xg.grad, x32.grad) <= 3e-2
    for n, w in zip(names, w32):
        assert rel_err(getattr(att, n).weight.grad, w.grad) <= 3e-2, n


# --------------------------------------------------------------------------- the whole block
@pytest.mark.parametrize("B,Hq,Hkv,L,D,pos,cap,dtype", [(2, 8, 2, 1, 128, 37, 64, torch.bfloat16),
                                                        (1, 4, 4, 5, 64, 0, 5, torch.bfloat16),
                                                        (3, 6, 2, 3, 128, 10, 13, torch.float32),
                                                        (1, 2, 1, 4, 6, 2, 9, torch.float32)])
def test_rope_append_equals_rope_then_copies(ops, gpu, B, Hq, Hkv, L, D, pos, cap, dtype):
    """The rotation that writes keys and values behind a cache: the bits of rope() followed by the two copies,
    with q, k, v as column ranges of one projection output (strided), and nothing else of the cache touched."""
    print("case rope_append", B, Hq, Hkv, L, D, pos, cap, dtype, flush=True)
    g = torch.Generator().manual_seed(77)
    qkv = torch.randn(B, L, Hq + 2 * Hkv, D, generator=g).to(dtype).to(gpu).transpose(1, 2)
    q, k, v = qkv[:, :Hq], qkv[:, Hq:Hq + Hkv], qkv[:, Hq + Hkv:]
    cos, sin = ops.rope_table(64, D, 10000.0, None, half=True)
    k_cache = torch.randn(B, Hkv, cap, D, generator=g).to(dtype).to(gpu)
    v_cache = torch.randn(B, Hkv, cap, D, generator=g).to(dtype).to(gpu)
    k_want, v_want = k_cache.clone(), v_cache.clone()
    q_ref, k_ref = ops.rope(q, k, cos, sin, 3)
    k_want[:, :, pos:pos + L] = k_ref
    v_want[:, :, pos:pos + L] = v
    q_out = ops.rope_append(q, k, v, cos, sin, k_cache, v_cache, pos, 3)
    assert torch.equal(q_out, q_ref) and torch.equal(k_cache, k_want) and torch.equal(v_cache, v_want)
    from adaptivetrainingsystem_amd._lib import AtsError
    with pytest.raises(AtsError):
        ops.rope_append(q, k, v, cos, sin, k_cache, v_cache, cap - L + 1, 3)


def test_gqa_module_cache_grows_in_place(gpu):
    """Decoding step after step: the cache handed back is the head of a buffer with room to grow, the next
    step writes its rows behind it without copying, and outputs and cache contents equal what concatenation
    gives (model.py:700-704).  Continuing twice from one cache, or from an older one, copies instead and
    leaves the other continuation's cache alone."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    hidden, nh, nkv, B, L = 512, 4, 2, 3, 70
    D = hidden // nh
    torch.manual_seed(16)
    att = A.GroupedQueryAttention(LayerConfig(hidden, 4 * hidden, 1, 1, num_heads=nh, num_kv_heads=nkv, seq_length=512))
    with torch.no_grad():
        for p in att.parameters():
            p.mul_(20.0)
    att = att.to(torch.bfloat16).to(gpu).eval()
    w = [getattr(att, n).weight.detach().cpu() for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
    x = torch.randn(B, L, hidden, generator=gen(120)).bfloat16()
    with torch.no_grad():
        _, cache = att(x.to(gpu), use_cache=True)
    _, ref_cache = O.gqa_forward(x, *w, nh, nkv, use_cache=True)
    ptrs = set()
    for step in range(6):
        x1 = torch.randn(B, 1, hidden, generator=gen(121 + step)).bfloat16()
        with torch.no_grad():
            plain = att(x1.to(gpu), past_key_value=cache)                    # concatenating path, no cache back
            o1, new_cache = att(x1.to(gpu), past_key_value=cache, use_cache=True)
        r1, ref_cache = O.gqa_forward(x1, *w, nh, nkv, past_key_value=ref_cache, use_cache=True)
        assert torch.equal(o1, plain) and rel_err(o1, r1) <= BF16_TOL
        assert new_cache[0].shape == (B, nkv, L + 1 + step, D) and new_cache[1].shape == new_cache[0].shape
        assert rel_err(new_cache[0], ref_cache[0]) <= BF16_TOL and rel_err(new_cache[1], ref_cache[1]) <= BF16_TOL
        assert torch.equal(new_cache[0][:, :, :L + step], cache[0]) and torch.equal(new_cache[1][:, :, :L + step], cache[1])
        cache = new_cache
        ptrs.add((cache[0].data_ptr(), cache[1].data_ptr()))
    assert len(ptrs) == 1                         # one buffer pair served all six steps
    # two continuations from the same state: the second one must not disturb the first one's new row
    xa = torch.randn(B, 1, hidden, generator=gen(130)).bfloat16().to(gpu)
    xb = torch.randn(B, 1, hidden, generator=gen(131)).bfloat16().to(gpu)
    with torch.no_grad():
        oa, cache_a = att(xa, past_key_value=cache, use_cache=True)
        keep_a = [t.clone() for t in cache_a]
        ob, cache_b = att(xb, past_key_value=cache, use_cache=True)
        oa2 = att(xa, past_key_value=cache)
        ob2 = att(xb, past_key_value=cache)
    assert torch.equal(cache_a[0], keep_a[0]) and torch.equal(cache_a[1], keep_a[1])
    assert torch.equal(oa, oa2) and torch.equal(ob, ob2) and not torch.equal(oa, ob)
    assert cache_b[0].data_ptr() != cache_a[0].data_ptr()
    # a chunk of several tokens on top of a cache, float32 cache tensors converted on the way in
    x4 = torch.randn(B, 4, hidden, generator=gen(132)).bfloat16().to(gpu)
    with torch.no_grad():
        o4, c4 = att(x4, past_key_value=(cache_b[0].float(), cache_b[1].float()), use_cache=True)
        o4_plain = att(x4, past_key_value=cache_b)
    assert torch.equal(o4, o4_plain) and c4[0].shape[2] == cache_b[0].shape[2] + 4 and c4[0].dtype == torch.bfloat16


# --------------------------------------------------------------------------- padding mask
def _padding_mask(B, Lk, seed, left=0):
    """Right padding of a different length per batch entry (every query keeps a real key in view),
    optionally with `left` padded keys in front as well."""
    g = gen(seed)
    mask = torch.ones(B, Lk)
    for b in range(B):
        n_real = int(torch.randint(max(1, Lk // 3), Lk + 1, (1,), generator=g))
        mask[b, n_real:] = 0
    mask[:, :left] = 0
    return mask


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D", [(2, 4, 2, 200, 200, 128), (3, 8, 2, 300, 300, 64), (1, 1, 1, 1, 1, 128),
                                             (2, 2, 2, 129, 129, 64), (2, 4, 1, 520, 520, 128), (2, 4, 2, 70, 300, 64),
                                             (3, 32, 8, 1, 513, 128), (2, 2, 1, 31, 31, 64), (1, 2, 1, 4099, 4200, 128)])
def test_causal_attention_padding_mask(ops, gpu, B, Hq, Hkv, L, Lk, D):
    """Forward and backward with (1 - mask) * -1e4 on the keys, against the oracle and autograd over it."""
    print("case attention padding mask", B, Hq, Hkv, L, Lk, D, flush=True)
    g = gen(111)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    mask = _padding_mask(B, Lk, 112)
    if Lk > L:
        mask[:, :Lk - L + 1] = 1        # the first query's keys (the cache and itself) hold a real one
    rep = Hq // Hkv
    q32, k32, v32 = (t.float().requires_grad_() for t in (q, k, v))
    ref = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5, mask)
    ref.backward(dout.float())
    bias = ((1.0 - mask) * -1e4).to(gpu)
    out, lse = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), return_lse=True, key_bias=bias)
    assert rel_err(out, ref) <= BF16_TOL
    s = torch.matmul(q.float(), k.repeat_interleave(rep, dim=1).float().transpose(-2, -1)) * D ** -0.5
    s = s.masked_fill(torch.triu(torch.ones(L, Lk, dtype=torch.bool), diagonal=1 + Lk - L), float("-inf"))
    assert rel_err(lse, torch.logsumexp(s + ((1.0 - mask) * -1e4)[:, None, None, :], -1)) <= 1e-4
    dq, dk, dv = ops.causal_attention_bwd(q.to(gpu), k.to(gpu), v.to(gpu), out, lse, dout.to(gpu), key_bias=bias)
    assert rel_err(dv, v32.grad) <= GRAD_TOL
    assert rel_err(dq, q32.grad) <= GRAD_TOL
    assert rel_err(dk, k32.grad) <= GRAD_TOL
    # padded keys receive no gradient at all
    padded = (mask == 0)[:, None, :, None].expand(B, Hkv, Lk, D)
    assert not dk.cpu()[padded].any() and not dv.cpu()[padded].any()
    # a mask of ones is the unmasked result up to the rounding of one fused multiply-add
    ones = torch.zeros(B, Lk, device=gpu)
    assert rel_err(ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), key_bias=ones),
                   ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu))) <= 1e-2


def test_attention_padding_mask_left_padding_and_errors(ops, gpu):
    """Left padding: queries that see a real key match the oracle; a query whose visible keys are all
    padded stays finite (there the reference spreads weight over keys behind the causal fill, which this
    kernel never reads).  Wrong bias shapes and dtypes are refused."""
    from adaptivetrainingsystem_amd import AtsError
    B, Hq, Hkv, L, D, left = 2, 4, 2, 150, 64, 70
    g = gen(113)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, L, D, generator=g).bfloat16()
    mask = torch.ones(B, L)
    mask[:, :left] = 0
    ref = O.attention_standard(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1), D ** -0.5, mask)
    bias = ((1.0 - mask) * -1e4).to(gpu)
    out = ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), key_bias=bias)
    assert torch.isfinite(out.float()).all()
    assert rel_err(out[:, left:], ref[:, left:]) <= BF16_TOL
    with pytest.raises(AtsError):
        ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), key_bias=bias[:, :-1])
    with pytest.raises(AtsError):
        ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), key_bias=bias.double())
    with pytest.raises(AtsError):
        ops.causal_attention(q.to(gpu), k.to(gpu), v.to(gpu), key_bias=bias.cpu())


def test_gqa_module_attention_mask(gpu):
    """attention_mask [batch, seq] through the module, forward and backward, float and integer masks."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    hidden, nh, nkv, B, L = 512, 4, 2, 3, 140
    torch.manual_seed(15)
    cfg = LayerConfig(hidden, 4 * hidden, 1, 1, num_heads=nh, num_kv_heads=nkv, seq_length=512)
    att = A.GroupedQueryAttention(cfg)
    with torch.no_grad():
        for p in att.parameters():
            p.mul_(20.0)
    att = att.to(torch.bfloat16).to(gpu).train()
    x = torch.randn(B, L, hidden, generator=gen(114)).bfloat16()
    dy = torch.randn(B, L, hidden, generator=gen(115)).bfloat16()
    mask = _padding_mask(B, L, 116)
    xg = x.to(gpu).requires_grad_()
    out = att(xg, mask.long().to(gpu))
    out.backward(dy.to(gpu))
    names = ("q_proj", "k_proj", "v_proj", "o_proj")
    w32 = [getattr(att, n).weight.detach().float().cpu().requires_grad_() for n in names]
    x32 = x.float().requires_grad_()
    ref = O.gqa_forward(x32, *w32, nh, nkv, attention_mask=mask)
    ref.backward(dy.float())
    assert rel_err(out, ref) <= BF16_TOL
    assert rel_err(xg.grad, x32.grad) <= 3e-2
    for n, w in zip(names, w32):
        assert rel_err(getattr(att, n).weight.grad, w.grad) <= 3e-2, n
    with torch.no_grad():
        assert torch.equal(att(x.to(gpu), mask.to(gpu)), out.detach())      # float mask, no-grad path
        assert not torch.equal(att(x.to(gpu)), out.detach())
    with torch.no_grad():       # a [B, 1, L, L] mask of ones masks nothing (up to the rounding of the added zeros)
        assert rel_err(att(x.to(gpu), torch.ones(B, 1, L, L, device=gpu)), att(x.to(gpu))) <= 1e-2
    with pytest.raises(A.AtsError):
        att(x.to(gpu), torch.ones(B, L + 1, device=gpu))
    # through a block: the mask reaches the attention sub-layer (model.py:1599)
    block = A.TransformerBlock(LayerConfig(hidden, 2 * hidden, 1, 1, num_heads=nh, num_kv_heads=nkv, seq_length=512,
                                           use_moe=False)).to(torch.bfloat16).to(gpu).eval()
    with torch.no_grad():
        y_masked, y_plain = block(x.to(gpu), mask.to(gpu)), block(x.to(gpu))
    y_masked = y_masked[0] if isinstance(y_masked, tuple) else y_masked
    y_plain = y_plain[0] if isinstance(y_plain, tuple) else y_plain
    n0 = int(mask[0].sum())
    assert torch.equal(y_masked[0, :n0], y_plain[0, :n0])          # real positions see no padded key anyway
    if n0 < L:
        assert not torch.equal(y_masked[0, n0:], y_plain[0, n0:])


def _oracle_block_dense(x, w, nh, nkv, eps):
    """model.py:1598-1611 with a dense SwiGLU FFN, from the oracle's pieces (float32 leaves)."""
    a = O.gqa_forward(O.rmsnorm(x, w["input_norm.weight"], eps), w["self_attn.q_proj.weight"],
                      w["self_attn.k_proj.weight"], w["self_attn.v_proj.weight"], w["self_attn.o_proj.weight"], nh, nkv)
    x1 = x + a
    return x1 + O.swiglu_expert(O.rmsnorm(x1, w["post_attn_norm.weight"], eps), w["ffn.gate_up_proj.weight"],
                                w["ffn.down_proj.weight"])


def test_transformer_block_dense_forward_backward(gpu):
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    hidden, nh, nkv, B, L = 256, 4, 2, 2, 96
    torch.manual_seed(15)
    cfg = LayerConfig(hidden, 512, 1, 1, num_heads=nh, num_kv_heads=nkv, seq_length=512, use_moe=False)
    blk = A.TransformerBlock(cfg)
    assert isinstance(blk.ffn, A.DenseSwiGLU) and isinstance(blk.self_attn, A.DenseGroupedQueryAttention)
    with torch.no_grad():
        for n, p in blk.named_parameters():
            if "norm" in n:
                p.add_(torch.randn(p.shape, generator=gen(102)) * 0.2)
            else:
                p.mul_(12.0)
    blk = blk.to(torch.bfloat16).to(gpu).train()
    x = torch.randn(B, L, hidden, generator=gen(103)).bfloat16()
    dy = torch.randn(B, L, hidden, generator=gen(104)).bfloat16()
    xg = x.to(gpu).requires_grad_()
    out, aux = blk(xg)
    assert aux is None and out.shape == x.shape
    out.backward(dy.to(gpu))
    w32 = {n: p.detach().float().cpu().requires_grad_() for n, p in blk.named_parameters()}
    x32 = x.float().requires_grad_()
    ref = _oracle_block_dense(x32, w32, nh, nkv, 1e-6)
    ref.backward(dy.float())
    assert rel_err(out, ref) <= BF16_TOL
    assert rel_err(xg.grad, x32.grad) <= 3e-2
    for n, p in blk.named_parameters():
        assert rel_err(p.grad, w32[n].grad) <= 3e-2, n
    # checkpointed forward recomputes through the same kernels: same gradients bit for bit
    blk.zero_grad()
    blk.gradient_checkpointing = True
    xg2 = x.to(gpu).requires_grad_()
    out2, _ = blk(xg2)
    out2.backward(dy.to(gpu))
    assert torch.equal(out2, out) and torch.equal(xg2.grad, xg.grad)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_transformer_block_dropout_with_and_without_checkpointing(gpu, dtype):
    """Attention dropout under gradient checkpointing: the recomputed forward must draw the mask of the first
    forward, or the saved output / log-sum-exp and the recomputed probabilities disagree and every gradient is
    silently wrong.  Same torch.manual_seed, once without and once with checkpointing: outputs and all
    gradients bit for bit; a different seed gives a different mask."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    hidden, nh, nkv, B, L = 256, 4, 2, 2, 96
    torch.manual_seed(21)
    cfg = LayerConfig(hidden, 512, 1, 1, num_heads=nh, num_kv_heads=nkv, seq_length=512, use_moe=False, dropout=0.25)
    blk = A.TransformerBlock(cfg)
    with torch.no_grad():
        for n, p in blk.named_parameters():
            if "norm" not in n:
                p.mul_(12.0)
    blk = blk.to(dtype).to(gpu).train()
    assert blk.self_attn.dropout_p == 0.25
    x = torch.randn(B, L, hidden, generator=gen(171)).to(dtype).to(gpu)
    dy = torch.randn(B, L, hidden, generator=gen(172)).to(dtype).to(gpu)

    def run(checkpointing, seed):
        blk.zero_grad()
        blk.gradient_checkpointing = checkpointing
        torch.manual_seed(seed)
        xg = x.clone().requires_grad_()
        out, _ = blk(xg)
        out.backward(dy)
        return out.detach(), xg.grad, {n: p.grad.clone() for n, p in blk.named_parameters()}

    out_a, dx_a, g_a = run(False, 99)
    out_b, dx_b, g_b = run(True, 99)
    assert torch.equal(out_a, out_b) and torch.equal(dx_a, dx_b)
    for n in g_a:
        assert torch.equal(g_a[n], g_b[n]), n
    out_c, _, _ = run(True, 100)
    assert not torch.equal(out_a, out_c)
    # the same mask whatever was constructed before: another attention module changes nothing
    A.GroupedQueryAttention(cfg)
    out_d, dx_d, _ = run(False, 99)
    assert torch.equal(out_a, out_d) and torch.equal(dx_a, dx_d)


def test_transformer_block_moe_composition_and_patterns(gpu):
    """The MoE block equals its own sub-modules composed by hand (the routing itself is checked against the oracle
    on bit-equal logits elsewhere), every parameter gets a finite gradient, and the layer patterns select as the
    reference's do."""
    import adaptivetrainingsystem_amd as A
    from adaptivetrainingsystem_amd.workloads import LayerConfig
    hidden, B, L = 256, 2, 64
    torch.manual_seed(16)
    cfg = LayerConfig(hidden, 384, 4, 2, num_heads=4, num_kv_heads=4, seq_length=256, use_moe=True, num_layers=8)
    blk = A.TransformerBlock(cfg).to(torch.bfloat16).to(gpu)
    assert blk.use_moe and isinstance(blk.ffn, A.MoEFFNLayer)
    blk.eval()
    x = torch.randn(B, L, hidden, generator=gen(105)).bfloat16().to(gpu)
    with torch.no_grad():
        out, aux = blk(x)
        x1 = x + blk.self_attn(blk.input_norm(x))
        f, aux2 = blk.ffn(blk.post_attn_norm(x1))
        assert torch.equal(out, x1 + f) and torch.equal(aux, aux2)
    blk.train()
    xg = x.clone().requires_grad_()
    out, aux = blk(xg)
    (out.float().pow(2).mean() + aux).backward()
    assert torch.isfinite(xg.grad).all()
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in blk.parameters())
    keys = set(blk.state_dict())
    assert {"input_norm.weight", "post_attn_norm.weight", "self_attn.q_proj.weight", "ffn.gate.weight",
            "ffn.experts.0.gate_up_proj.weight", "ffn.experts.3.down_proj.weight"} <= keys
    sel = lambda pattern, **kw: [i for i in range(8) if A.TransformerBlock._should_use_moe(
        i, LayerConfig(8, 8, 2, 1, use_moe=True, num_layers=8, moe_pattern=pattern, **kw))]
    assert sel("all") == list(range(8)) and sel("none") == []
    assert sel("every_3rd") == [2, 5] and sel("every_4th") == [3, 7]
    assert sel("sandwich") == [2, 3, 4, 5] and sel("sandwich", dense_start_layers=1, dense_end_layers=3) == [1, 2, 3, 4]
    assert sel(lambda i, n: i % 2 == 0) == [0, 2, 4, 6]


# --------------------------------------------------------------------------- per-query masks and dropout
def _pair_mask(B, L, Lk, seed, p_zero=0.3):
    """[B, 1, L, Lk] of ones and zeros in which every query keeps its own position (so no row is masked out
    entirely: a fully masked row falls back on the -1e4 constants, which float32 scores cannot resolve)."""
    m = (torch.rand(B, 1, L, Lk, generator=gen(seed)) >= p_zero).float()
    i = torch.arange(L)
    m[:, 0, i, i + (Lk - L)] = 1.0
    return m


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D", [(2, 4, 2, 200, 200, 128), (1, 8, 2, 300, 300, 64), (1, 1, 1, 1, 1, 128),
                                             (2, 3, 3, 129, 129, 64), (1, 4, 1, 520, 520, 128), (2, 4, 2, 70, 300, 64),
                                             (1, 2, 1, 31, 31, 64), (1, 2, 2, 130, 131, 128)])
def test_causal_attention_pair_mask(ops, gpu, B, Hq, Hkv, L, Lk, D):
    """[B, 1, L, Lk] masks (model.py:819-824 with a 4-D mask): forward, log-sum-exp and the three gradients
    against the oracle and autograd over it; a 4-D mask that repeats a [B, Lk] mask for every query gives what
    the per-key path gives; one matrix shared by the batch."""
    print("case attention pair mask", B, Hq, Hkv, L, Lk, D, flush=True)
    g = gen(131)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    mask = _pair_mask(B, L, Lk, 132)
    rep = Hq // Hkv
    q32, k32, v32 = (t.float().requires_grad_() for t in (q, k, v))
    ref = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5, mask)
    ref.backward(dout.float())
    bias = ((1.0 - mask[:, 0]) * -1e4).to(gpu)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    out, lse = ops.causal_attention(qg, kg, vg, return_lse=True, pair_bias=bias)
    assert rel_err(out, ref) <= BF16_TOL
    s = torch.matmul(q.float(), k.repeat_interleave(rep, dim=1).float().transpose(-2, -1)) * D ** -0.5
    s = s.masked_fill(torch.triu(torch.ones(L, Lk, dtype=torch.bool), diagonal=1 + Lk - L), float("-inf"))
    assert rel_err(lse, torch.logsumexp(s + (1.0 - mask) * -1e4, -1)) <= 1e-4
    dq, dk, dv = ops.causal_attention_bwd(qg, kg, vg, out, lse, dout.to(gpu), pair_bias=bias)
    assert rel_err(dv, v32.grad) <= GRAD_TOL
    assert rel_err(dq, q32.grad) <= GRAD_TOL
    assert rel_err(dk, k32.grad) <= GRAD_TOL
    # the per-key mask written as a 4-D mask, alone and on top of a per-key bias
    pad = _padding_mask(B, Lk, 133)
    pad[:, :Lk - L + 1] = 1
    kb = ((1.0 - pad) * -1e4).to(gpu)
    per_key = ops.causal_attention(qg, kg, vg, key_bias=kb)
    as_pair = ops.causal_attention(qg, kg, vg, pair_bias=kb[:, None, :].expand(B, L, Lk).contiguous())
    assert rel_err(as_pair, per_key) <= 1e-2
    both = ops.causal_attention(qg, kg, vg, key_bias=kb, pair_bias=torch.zeros(1, L, Lk, device=gpu))
    assert torch.equal(both, as_pair)
    # one matrix for the whole batch
    shared = ops.causal_attention(qg, kg, vg, pair_bias=bias[:1])
    assert torch.equal(shared[:1], out[:1])


def _head_mask(B, H, L, Lk, seed, p_zero=0.3):
    """[B, H, L, Lk] of ones and zeros, a different pattern per head; every query keeps its own position."""
    m = (torch.rand(B, H, L, Lk, generator=gen(seed)) >= p_zero).float()
    i = torch.arange(L)
    m[:, :, i, i + (Lk - L)] = 1.0
    return m


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D", [(2, 4, 2, 200, 200, 128), (1, 8, 2, 300, 300, 64), (2, 3, 3, 129, 129, 64),
                                             (2, 4, 1, 70, 300, 64), (1, 2, 2, 130, 131, 128)])
def test_causal_attention_mask_per_head(ops, gpu, B, Hq, Hkv, L, Lk, D):
    """[B, H, L, Lk] masks, which the reference's broadcast (model.py:819-824) accepts like any mask that expands
    to the scores: forward, log-sum-exp and the three gradients (dK / dV sum over the query heads of a kv head,
    each with its own mask) against the oracle and autograd over it; a per-head mask that repeats one matrix
    equals the shared form bit for bit; one set of head masks shared by the batch."""
    print("case attention head mask", B, Hq, Hkv, L, Lk, D, flush=True)
    g = gen(171)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    mask = _head_mask(B, Hq, L, Lk, 172)
    rep = Hq // Hkv
    q32, k32, v32 = (t.float().requires_grad_() for t in (q, k, v))
    ref = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5, mask)
    ref.backward(dout.float())
    bias = ((1.0 - mask) * -1e4).to(gpu)
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    out, lse = ops.causal_attention(qg, kg, vg, return_lse=True, pair_bias=bias)
    assert rel_err(out, ref) <= BF16_TOL
    s = torch.matmul(q.float(), k.repeat_interleave(rep, dim=1).float().transpose(-2, -1)) * D ** -0.5
    s = s.masked_fill(torch.triu(torch.ones(L, Lk, dtype=torch.bool), diagonal=1 + Lk - L), float("-inf"))
    assert rel_err(lse, torch.logsumexp(s + (1.0 - mask) * -1e4, -1)) <= 1e-4
    dq, dk, dv = ops.causal_attention_bwd(qg, kg, vg, out, lse, dout.to(gpu), pair_bias=bias)
    assert rel_err(dv, v32.grad) <= GRAD_TOL
    assert rel_err(dq, q32.grad) <= GRAD_TOL
    assert rel_err(dk, k32.grad) <= GRAD_TOL
    # the same matrix for every head: the shared form's bits
    one = bias[:, :1].contiguous()
    shared = ops.causal_attention(qg, kg, vg, pair_bias=one)
    repeated = ops.causal_attention(qg, kg, vg, pair_bias=one.expand(B, Hq, L, Lk).contiguous())
    assert torch.equal(shared, repeated)
    # head masks shared by the batch
    first = ops.causal_attention(qg, kg, vg, pair_bias=bias[:1])
    assert torch.equal(first[:1], out[:1])
    # float32 route
    if D % 4 == 0 and L <= 200:
        q32, k32, v32 = (t.float().requires_grad_() for t in (q, k, v))
        ref = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5, mask)
        ref.backward(dout.float())
        o32, state = ops.attention_f32(qg.float(), kg.float(), vg.float(), pair_bias=bias, return_weights=True)
        assert rel_err(o32, ref) <= F32_TOL
        dq, dk, dv = ops.attention_f32_bwd(state, dout.float().to(gpu), B, Hq, Hkv, L, Lk, D, None, 0.0, 0)
        assert rel_err(dq, q32.grad) <= F32_TOL and rel_err(dk, k32.grad) <= F32_TOL and rel_err(dv, v32.grad) <= F32_TOL
    with pytest.raises(Exception):
        ops.causal_attention(qg, kg, vg, pair_bias=torch.zeros(B, Hq + 1, L, Lk, device=gpu))


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D,p", [(2, 4, 2, 200, 200, 128, 0.25), (1, 8, 2, 300, 300, 64, 0.1),
                                               (2, 3, 3, 129, 129, 64, 0.5), (1, 4, 1, 520, 520, 128, 0.3),
                                               (2, 4, 2, 70, 300, 64, 0.25), (1, 2, 1, 31, 31, 64, 0.9)])
def test_causal_attention_dropout(ops, gpu, B, Hq, Hkv, L, Lk, D, p):
    """Dropout on the attention weights (model.py:831-833).  The kernels' keep / drop decisions are a function of
    (seed, batch, head, query, key) that the oracle restates on the CPU; with that mask made explicit the
    oracle's forward and autograd over it are the reference for output and gradients.  The log-sum-exp is that
    of the undropped scores; another seed gives another mask; p = 0 is the plain kernel's result."""
    print("case attention dropout", B, Hq, Hkv, L, Lk, D, p, flush=True)
    g = gen(141)
    q = torch.randn(B, Hq, L, D, generator=g).bfloat16()
    k = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    v = torch.randn(B, Hkv, Lk, D, generator=g).bfloat16()
    dout = torch.randn(B, L, Hq * D, generator=g).bfloat16()
    seed = 0x5DEECE66D1234567
    keep = O.attention_dropout_keep(seed, B, Hq, L, Lk, p)
    rep = Hq // Hkv
    q32, k32, v32 = (t.float().requires_grad_() for t in (q, k, v))
    ref = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5,
                               dropout_keep=keep, dropout_p=p)
    ref.backward(dout.float())
    qg, kg, vg = q.to(gpu), k.to(gpu), v.to(gpu)
    out, lse = ops.causal_attention(qg, kg, vg, return_lse=True, dropout_p=p, dropout_seed=seed)
    assert rel_err(out, ref) <= BF16_TOL
    plain, lse_plain = ops.causal_attention(qg, kg, vg, return_lse=True)
    assert rel_err(lse, lse_plain) <= 1e-5
    dq, dk, dv = ops.causal_attention_bwd(qg, kg, vg, out, lse, dout.to(gpu), dropout_p=p, dropout_seed=seed)
    assert rel_err(dv, v32.grad) <= GRAD_TOL
    assert rel_err(dq, q32.grad) <= GRAD_TOL
    assert rel_err(dk, k32.grad) <= GRAD_TOL
    other = ops.causal_attention(qg, kg, vg, dropout_p=p, dropout_seed=seed + 1)
    if L > 1:
        assert not torch.equal(other, out)
    assert torch.equal(ops.causal_attention(qg, kg, vg, dropout_p=p, dropout_seed=seed), out)      # reproducible
    # with a padding mask on top (folded into the pair bias by the host)
    pad = _padding_mask(B, Lk, 142)
    pad[:, :Lk - L + 1] = 1
    ref_m = O.attention_standard(q.float(), k.float().repeat_interleave(rep, dim=1),
                                 v.float().repeat_interleave(rep, dim=1), D ** -0.5, pad, dropout_keep=keep, dropout_p=p)
    out_m = ops.causal_attention(qg, kg, vg, key_bias=((1.0 - pad) * -1e4).to(gpu), dropout_p=p, dropout_seed=seed)
    assert rel_err(out_m, ref_m) <= BF16_TOL


def test_attention_extras_errors(ops, gpu):
    q = torch.randn(1, 2, 8, 64, device=gpu).bfloat16()
    from adaptivetrainingsystem_amd._lib import AtsError
    with pytest.raises(AtsError):
        ops.causal_attention(q, q, q, dropout_p=1.0)
    with pytest.raises(AtsError):
        ops.causal_attention(q, q, q, pair_bias=torch.zeros(1, 8, 9, device=gpu))
    with pytest.raises(AtsError):
        ops.causal_attention(q, q, q, pair_bias=torch.zeros(1, 8, 8, device=gpu, dtype=torch.float64))


def test_gqa_module_pair_mask_and_dropout(gpu):
    """GroupedQueryAttention with a [B, 1, L, L] mask and with config.dropout > 0 in training mode, against the
    oracle's gqa_forward / attention_standard (model.py:663-731, 819-833)."""
    from types import SimpleNamespace
    from adaptivetrainingsystem_amd.layers import GroupedQueryAttention
    from adaptivetrainingsystem_amd._lib import AtsError
    hidden, nh, nkv, B, L = 256, 4, 2, 2, 96
    torch.manual_seed(5)
    cfg = SimpleNamespace(hidden_size=hidden, num_heads=nh, num_kv_heads=nkv, seq_length=256, dropout=0.2)
    att = GroupedQueryAttention(cfg).to(gpu).bfloat16()
    w = [getattr(att, n).weight.detach().cpu() for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
    x = torch.randn(B, L, hidden, generator=gen(151)).bfloat16()
    mask = _pair_mask(B, L, L, 152)
    att.eval()
    with torch.no_grad():
        out = att(x.to(gpu), attention_mask=mask.to(gpu))
    assert rel_err(out, O.gqa_forward(x, *w, nh, nkv, attention_mask=mask)) <= BF16_TOL
    # one mask per head (the reference's broadcast takes any mask that expands to [B, H, L, L]); a wrong head count raises
    hmask = _head_mask(B, nh, L, L, 153)
    with torch.no_grad():
        out_h = att(x.to(gpu), attention_mask=hmask.to(gpu))
    assert rel_err(out_h, O.gqa_forward(x, *w, nh, nkv, attention_mask=hmask)) <= BF16_TOL
    with pytest.raises(AtsError):
        att(x.to(gpu), attention_mask=torch.ones(B, nh + 1, L, L, device=gpu))
    # eval mode: dropout is off (model.py:832)
    with torch.no_grad():
        plain = att(x.to(gpu))
    assert rel_err(plain, O.gqa_forward(x, *w, nh, nkv)) <= BF16_TOL
    # training mode: a fresh mask per call, the one the recorded seed describes
    att.train()
    with torch.no_grad():
        d1 = att(x.to(gpu))
        seed1 = att._state["last_dropout_seed"]
        d2 = att(x.to(gpu))
    assert not torch.equal(d1, d2) and not torch.equal(d1, plain)
    D = hidden // nh
    keep = O.attention_dropout_keep(seed1, B, nh, L, L, 0.2)
    lin = lambda a, m: torch.nn.functional.linear(a.float(), m.float()).to(a.dtype)
    qh = lin(x, w[0]).view(B, L, nh, D).transpose(1, 2)
    kh = lin(x, w[1]).view(B, L, nkv, D).transpose(1, 2)
    vh = lin(x, w[2]).view(B, L, nkv, D).transpose(1, 2)
    cos, sin = O.rope_table(L, D, 10000.0)
    qh, kh = O.rope_apply(qh, kh, cos, sin)
    a = O.attention_standard(qh, kh.repeat_interleave(nh // nkv, dim=1), vh.repeat_interleave(nh // nkv, dim=1), D ** -0.5,
                             dropout_keep=keep, dropout_p=0.2)
    assert rel_err(d1, lin(a, w[3]).view(B, L, hidden)) <= BF16_TOL
    # gradients flow through the dropped attention
    xg = x.to(gpu).requires_grad_()
    att(xg).float().sum().backward()
    assert xg.grad is not None and torch.isfinite(xg.grad).all() and att.q_proj.weight.grad is not None


# --------------------------------------------------------------------------- float32
F32_TOL = 2e-4       # float32 products with float32 accumulation, relative to the oracle's max-abs


@pytest.mark.parametrize("B,Hq,Hkv,L,Lk,D,p", [(2, 4, 2, 64, 64, 64, 0.0), (1, 8, 2, 130, 130, 128, 0.0),
                                               (2, 3, 3, 33, 70, 32, 0.0), (1, 1, 1, 1, 1, 64, 0.0),
                                               (2, 4, 1, 50, 50, 64, 0.3), (1, 2, 2, 17, 29, 96, 0.5)])
def test_attention_float32(ops, gpu, B, Hq, Hkv, L, Lk, D, p):
    """_standard_attention on float32 tensors (model.py:807-839): output and the three gradients against the
    oracle and autograd over it, with a padding mask, a [B, 1, L, Lk] mask and dropout."""
    print("case attention float32", B, Hq, Hkv, L, Lk, D, p, flush=True)
    g = gen(161)
    q = torch.randn(B, Hq, L, D, generator=g)
    k = torch.randn(B, Hkv, Lk, D, generator=g)
    v = torch.randn(B, Hkv, Lk, D, generator=g)
    dout = torch.randn(B, L, Hq * D, generator=g)
    rep = Hq // Hkv
    seed = 77
    keep = O.attention_dropout_keep(seed, B, Hq, L, Lk, p) if p > 0 else None
    pad = _padding_mask(B, Lk, 162)
    pad[:, :Lk - L + 1] = 1
    pair = _pair_mask(B, L, Lk, 163)
    for mask, kw in ((None, {}), (pad, {"key_bias": ((1.0 - pad) * -1e4).to(gpu)}),
                     (pair, {"pair_bias": ((1.0 - pair[:, 0]) * -1e4).to(gpu)})):
        q32, k32, v32 = (t.clone().requires_grad_() for t in (q, k, v))
        ref = O.attention_standard(q32, k32.repeat_interleave(rep, dim=1), v32.repeat_interleave(rep, dim=1), D ** -0.5,
                                   mask, dropout_keep=keep, dropout_p=p)
        ref.backward(dout)
        out, state = ops.attention_f32(q.to(gpu), k.to(gpu), v.to(gpu), dropout_p=p, dropout_seed=seed, return_weights=True,
                                       **kw)
        assert out.shape == (B, L, Hq * D) and out.dtype == torch.float32
        assert rel_err(out, ref) <= F32_TOL
        dq, dk, dv = ops.attention_f32_bwd(state, dout.to(gpu), B, Hq, Hkv, L, Lk, D, None, p, seed)
        assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
        assert rel_err(dv, v32.grad) <= F32_TOL
        assert rel_err(dq, q32.grad) <= F32_TOL
        assert rel_err(dk, k32.grad) <= F32_TOL


def test_gqa_module_float32(gpu):
    """GroupedQueryAttention on float32 activations and weights (the reference's CPU-runnable precision):
    forward against the oracle, gradients against autograd over it."""
    from types import SimpleNamespace
    from adaptivetrainingsystem_amd.layers import GroupedQueryAttention
    hidden, nh, nkv, B, L = 128, 4, 2, 2, 40
    torch.manual_seed(6)
    att = GroupedQueryAttention(SimpleNamespace(hidden_size=hidden, num_heads=nh, num_kv_heads=nkv, seq_length=64)).to(gpu)
    names = ("q_proj", "k_proj", "v_proj", "o_proj")
    w = [getattr(att, n).weight.detach().cpu().clone().requires_grad_() for n in names]
    x = torch.randn(B, L, hidden, generator=gen(171))
    mask = _padding_mask(B, L, 172)
    mask[:, 0] = 1
    xr = x.clone().requires_grad_()
    ref = O.gqa_forward(xr, *w, nh, nkv, attention_mask=mask)
    ref.square().sum().backward()
    xg = x.to(gpu).requires_grad_()
    out = att(xg, attention_mask=mask.to(gpu))
    assert out.dtype == torch.float32 and rel_err(out, ref) <= F32_TOL
    out.square().sum().backward()
    assert rel_err(xg.grad, xr.grad) <= 5 * F32_TOL
    for n, wr in zip(names, w):
        assert rel_err(getattr(att, n).weight.grad, wr.grad) <= 5 * F32_TOL, n
    with torch.no_grad():
        assert rel_err(att(x.to(gpu), attention_mask=mask.to(gpu)), ref) <= F32_TOL
