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
                                          (2, 3, 3, 129, 64), (1, 4, 1, 1024, 128), (1, 2, 2, 31, 64)])
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
    with pytest.raises(A.AtsError):
        att(x.to(gpu).requires_grad_())
