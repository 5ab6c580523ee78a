"""The reference's launcher names, called through ctypes exactly as the reference's wrapper calls them
(Src/Main_Scripts/core/cuda_opt_wrapper.py:98-108 RMSNorm, 156-169 RoPE apply, 219-228 SwiGLU, 337-344 RoPE
precompute: bare CDLL handle, every argument wrapped in a ctypes type, stream as c_void_p), compared with the
oracle.  float32 only, as those signatures are."""
import ctypes
import math

import pytest
import torch

from oracle import sparse_layer_oracle as O

pytestmark = pytest.mark.gpu


def gen(seed):
    return torch.Generator().manual_seed(seed)


@pytest.fixture(scope="module")
def raw(gpu):
    from adaptivetrainingsystem_amd import _lib
    _lib.load()
    return ctypes.CDLL(_lib.LIB_PATH), _lib.load()


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def test_rms_norm_launcher(raw, gpu):
    lib, typed = raw
    x = torch.randn(37, 520, generator=gen(1)) * 2.0
    w = torch.randn(520, generator=gen(2)) * 0.1 + 1.0
    xg, wg = x.to(gpu), w.to(gpu)
    out = torch.empty_like(xg)
    lib.rms_norm_launcher(ctypes.c_void_p(xg.data_ptr()), ctypes.c_void_p(wg.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                          ctypes.c_int(37), ctypes.c_int(520), ctypes.c_float(1e-6), _stream())
    torch.cuda.synchronize()
    assert typed.ats_legacy_last_status() == 0
    ref = O.rmsnorm(x, w, 1e-6)
    assert (out.cpu() - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()


def test_rope_launchers(raw, gpu):
    lib, typed = raw
    B, nH, L, D, max_seq, off, theta = 2, 3, 21, 64, 64, 5, 10000.0
    cos = torch.empty(max_seq, D // 2, device=gpu)
    sin = torch.empty(max_seq, D // 2, device=gpu)
    lib.rope_precompute_launcher(ctypes.c_void_p(cos.data_ptr()), ctypes.c_void_p(sin.data_ptr()), ctypes.c_int(max_seq),
                                 ctypes.c_int(D), ctypes.c_float(theta), _stream())
    torch.cuda.synchronize()
    assert typed.ats_legacy_last_status() == 0
    ch, sh = O.fused_rope_table(max_seq, D, theta)      # float32 evaluation; the kernel rounds the float64 value
    assert (cos.cpu() - ch).abs().max().item() <= 2e-5 and (sin.cpu() - sh).abs().max().item() <= 2e-5
    for pos, d in ((1, 0), (7, 3), (63, 31)):
        ang = pos * theta ** (-2.0 * d / D)
        assert abs(cos[pos, d].item() - math.cos(ang)) <= 1.2e-7 and abs(sin[pos, d].item() - math.sin(ang)) <= 1.2e-7
    q = torch.randn(B, nH, L, D, generator=gen(3))
    k = torch.randn(B, nH, L, D, generator=gen(4))
    qg, kg = q.to(gpu).clone(), k.to(gpu).clone()        # the launcher rotates in place (cuda_opt_wrapper.py:153-154)
    lib.rope_apply_launcher(ctypes.c_void_p(qg.data_ptr()), ctypes.c_void_p(kg.data_ptr()), ctypes.c_void_p(cos.data_ptr()),
                            ctypes.c_void_p(sin.data_ptr()), ctypes.c_int(B), ctypes.c_int(nH), ctypes.c_int(L),
                            ctypes.c_int(D), ctypes.c_int(off), _stream())
    torch.cuda.synchronize()
    assert typed.ats_legacy_last_status() == 0
    rq, rk = O.fused_rope_apply(q, k, cos.cpu(), sin.cpu(), off)
    assert torch.equal(qg.cpu(), rq) and torch.equal(kg.cpu(), rk)      # same table, same roundings: same bits


def test_swiglu_launcher(raw, gpu):
    lib, typed = raw
    T, I = 19, 1408
    gate = torch.randn(T, I, generator=gen(5))
    up = torch.randn(T, I, generator=gen(6)) * 2.0
    gg, ug = gate.to(gpu), up.to(gpu)
    out = torch.empty_like(gg)
    lib.swiglu_launcher(ctypes.c_void_p(gg.data_ptr()), ctypes.c_void_p(ug.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                        ctypes.c_int(T), ctypes.c_int(I), _stream())
    torch.cuda.synchronize()
    assert typed.ats_legacy_last_status() == 0
    ref = gate * torch.nn.functional.silu(up)            # cuda_opt_wrapper.py:476-478 convention: gate * silu(up)
    assert (out.cpu() - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()


@pytest.mark.parametrize("T,H,I", [(19, 512, 1408), (300, 264, 100), (1, 64, 4)])
def test_swiglu_fused_launcher(raw, gpu, T, H, I):
    """transformer_ops.cu:268-313, 411-434: (x . gate_w^T) * silu(x . up_w^T) in float32; the biases are accepted
    and, as in the original, not applied."""
    lib, typed = raw
    g = gen(7)
    x = torch.randn(T, H, generator=g)
    wg = torch.randn(I, H, generator=g) * 0.1
    wu = torch.randn(I, H, generator=g) * 0.1
    bias = torch.randn(I, generator=g)
    xg, wgg, wug, bg = x.to(gpu), wg.to(gpu), wu.to(gpu), bias.to(gpu)
    out = torch.full((T, I), 9.0, device=gpu)
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    lib.swiglu_fused_launcher(p(xg), p(wgg), p(wug), p(bg), p(bg), p(out), ctypes.c_int(T), ctypes.c_int(H),
                              ctypes.c_int(I), ctypes.c_bool(True), _stream())
    torch.cuda.synchronize()
    assert typed.ats_legacy_last_status() == 0
    ref = (x.double() @ wg.double().T) * torch.nn.functional.silu(x.double() @ wu.double().T)
    assert (out.cpu().double() - ref).abs().max().item() <= 1e-5 * ref.abs().max().item()
    # sizes that do not describe 16-byte rows are refused with a status, not a crash
    lib.swiglu_fused_launcher(p(xg), p(wgg), p(wug), None, None, p(out), ctypes.c_int(1), ctypes.c_int(H - 1),
                              ctypes.c_int(I), ctypes.c_bool(False), _stream())
    assert typed.ats_legacy_last_status() != 0


def test_fused_cross_entropy_accuracy_launcher(raw, gpu):
    """training/fused_loss.cu:183-193 as training/cuda_kernels.py:154-175 calls it: the three device scalars hold
    the sum of token losses, the number of correct predictions and the number of valid tokens."""
    lib, typed = raw
    T, V, pad = 37, 1000, -100
    g = gen(201)
    logits = torch.randn(T, V, generator=g) * 3
    labels = torch.randint(0, V, (T,), generator=g)
    labels[[3, 11]] = pad
    labels[20] = V + 5                       # outside the vocabulary: skipped as well (fused_loss.cu:82)
    labels[5] = logits[5].argmax()           # a certainly correct prediction
    ref = O.fused_loss(logits, labels, None, pad)
    lg, lb = logits.to(gpu), labels.to(gpu)
    loss = torch.full((1,), 7.0, device=gpu)             # the launcher clears its outputs (fused_loss.cu:195-197)
    acc = torch.full((1,), 7.0, device=gpu)
    valid = torch.full((1,), 7, dtype=torch.int64, device=gpu)
    lib.fused_cross_entropy_accuracy_launcher(ctypes.c_void_p(lg.data_ptr()), ctypes.c_void_p(lb.data_ptr()),
                                              ctypes.c_int64(pad), ctypes.c_void_p(loss.data_ptr()),
                                              ctypes.c_void_p(acc.data_ptr()), ctypes.c_void_p(valid.data_ptr()),
                                              ctypes.c_int(T), ctypes.c_int(V), _stream())
    torch.cuda.synchronize()
    assert typed.ats_legacy_last_status() == 0
    n = int(valid.item())
    assert n == T - 3
    assert abs(loss.item() / n - float(ref["loss"])) <= 1e-5 * max(1.0, abs(float(ref["loss"])))
    assert abs(acc.item() / n - float(ref["accuracy"])) <= 1e-6
    # nothing to do is not an error and clears the outputs
    lib.fused_cross_entropy_accuracy_launcher(ctypes.c_void_p(lg.data_ptr()), ctypes.c_void_p(lb.data_ptr()),
                                              ctypes.c_int64(pad), ctypes.c_void_p(loss.data_ptr()),
                                              ctypes.c_void_p(acc.data_ptr()), ctypes.c_void_p(valid.data_ptr()),
                                              ctypes.c_int(0), ctypes.c_int(V), _stream())
    torch.cuda.synchronize()
    assert typed.ats_legacy_last_status() == 0 and loss.item() == 0 and valid.item() == 0


def test_fused_grad_clip_launcher(raw, gpu):
    """training/fused_grad_clip.cu:117-175 as training/cuda_kernels.py:320-349 calls it: device arrays of float32
    gradient pointers and int32 sizes, the norm comes back as the return value."""
    lib, typed = raw
    lib.fused_grad_clip_launcher.restype = ctypes.c_float          # cuda_kernels.py:77
    g = gen(202)
    shapes = [(300, 70), (5,), (1,), (129, 33), (40000,)]
    for max_norm in (0.5, 1e6):
        grads = [torch.randn(*s, generator=g) for s in shapes]
        want_norm, want = O.clip_grad_norm([t.clone() for t in grads], max_norm)
        dev = [t.to(gpu) for t in grads]
        ptrs = torch.tensor([t.data_ptr() for t in dev], dtype=torch.int64, device=gpu)
        sizes = torch.tensor([t.numel() for t in dev], dtype=torch.int32, device=gpu)
        norm = lib.fused_grad_clip_launcher(ctypes.c_void_p(ptrs.data_ptr()), ctypes.c_void_p(sizes.data_ptr()),
                                            ctypes.c_int(len(dev)), ctypes.c_float(max_norm), _stream())
        torch.cuda.synchronize()
        assert typed.ats_legacy_last_status() == 0
        assert abs(norm - float(want_norm)) <= 1e-5 * float(want_norm)
        for got, ref in zip(dev, want):
            assert torch.allclose(got.cpu(), ref, rtol=1e-5, atol=1e-7)
    assert lib.fused_grad_clip_launcher(ctypes.c_void_p(0), ctypes.c_void_p(0), ctypes.c_int(0), ctypes.c_float(1.0),
                                        _stream()) == 0.0
