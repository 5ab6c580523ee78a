"""Parity of the fused cross-entropy and gradient-clipping kernels against the CPU oracle
(restatements of the reference's FusedLoss / clip_grad_norm_ PyTorch paths), through the C ABI."""
import pytest
import torch

from oracle import sparse_layer_oracle as O

pytestmark = pytest.mark.gpu


def rel_err(got, ref) -> float:
    got, ref = got.detach().double().cpu(), ref.detach().double().cpu()
    denom = ref.abs().max().item()
    return (got - ref).abs().max().item() / (denom if denom > 0 else 1.0)


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.fixture(scope="module")
def T_(gpu):
    from adaptivetrainingsystem_amd import _lib, training
    _lib.load()
    return training


@pytest.mark.parametrize("shape,V", [((4, 33), 1000), ((257,), 32000), ((3, 5), 37), ((16,), 50257), ((1,), 8)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("weighted", [False, True])
def test_fused_loss_forward_and_gradient(T_, gpu, shape, V, dtype, weighted):
    print("case fused_loss", shape, V, dtype, weighted, flush=True)
    g = gen(71)
    logits = (torch.randn(*shape, V, generator=g) * 2.5).to(dtype)
    labels = torch.randint(0, V, shape, generator=g)
    flat = labels.view(-1)
    if flat.numel() > 4:
        flat[1] = -100
        flat[3] = V + 7
    w = torch.rand(shape, generator=g) if weighted else None
    lg_ref = logits.float().clone().requires_grad_()
    ref = O.fused_loss(lg_ref, labels, w)
    (ref["loss"] * 1.7).backward()
    lg = logits.to(gpu).requires_grad_()
    out = T_.FusedLoss()(lg, labels.to(gpu), None if w is None else w.to(gpu))
    (out["loss"] * 1.7).backward()
    assert abs(out["loss"].item() - ref["loss"].item()) <= 1e-5 * max(1.0, abs(ref["loss"].item()))
    assert abs(out["raw_loss"].item() - ref["raw_loss"].item()) <= 1e-5 * max(1.0, abs(ref["raw_loss"].item()))
    assert out["valid_tokens"].item() == ref["valid_tokens"].item()
    assert abs(out["accuracy"].item() - ref["accuracy"].item()) <= 1e-6
    assert abs(out["perplexity"].item() - ref["perplexity"].item()) <= 1e-4 * ref["perplexity"].item()
    assert lg.grad.dtype == dtype and lg.grad.shape == logits.shape
    assert rel_err(lg.grad, lg_ref.grad) <= (1e-5 if dtype == torch.float32 else 2e-2)


def test_fused_loss_all_ignored_and_ties(T_, gpu):
    V = 64
    z = torch.zeros(6, V, device=gpu)
    out = T_.FusedLoss()(z, torch.full((6,), -100, device=gpu))
    assert out["loss"].item() == 0.0 and out["valid_tokens"].item() == 0 and torch.isinf(out["perplexity"]).item()
    # all logits equal: the arg-max is index 0
    labels = torch.tensor([0, 1, 0, 5, 0, 63], device=gpu)
    out = T_.FusedLoss()(z, labels)
    assert abs(out["accuracy"].item() - 0.5) < 1e-6
    assert abs(out["loss"].item() - torch.log(torch.tensor(float(V))).item()) < 1e-6


@pytest.mark.parametrize("max_norm", [1.0, 1e6])
@pytest.mark.parametrize("dtypes", [(torch.float32,), (torch.bfloat16,), (torch.float32, torch.bfloat16)])
def test_grad_norm_and_clip(T_, gpu, max_norm, dtypes):
    print("case grad clip", max_norm, dtypes, flush=True)
    g = gen(72)
    shapes = [(300, 257), (70001,), (3, 5, 7), (1,), (131072,), (65536,), (0,), (129, 1023)]
    grads = [(torch.randn(*s, generator=g) * (0.1 + i)).to(dtypes[i % len(dtypes)]) for i, s in enumerate(shapes)]
    ref_norm, ref_clipped = O.clip_grad_norm(grads, max_norm)
    params = []
    for x in grads:
        p = torch.nn.Parameter(torch.zeros(x.shape, dtype=x.dtype, device=gpu))
        p.grad = x.to(gpu)
        params.append(p)
    params.append(torch.nn.Parameter(torch.zeros(3, device=gpu)))      # no gradient: skipped
    clip = T_.FusedGradClip()
    norm = clip(params, max_norm)
    assert isinstance(norm, float) and abs(norm - ref_norm.item()) <= 2e-5 * ref_norm.item()
    for p, c in zip(params, ref_clipped):
        if c.numel():
            assert rel_err(p.grad, c) <= (1e-5 if c.dtype == torch.float32 else 1e-2)
    t = clip.norm_and_clip(params[:3], max_norm, clip=False)           # norm only, stays on the device
    assert t.is_cuda and t.dim() == 0
