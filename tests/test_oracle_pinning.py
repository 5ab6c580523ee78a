"""Pins the CPU oracle against things that do not share its code: float64 closed
forms, library routines, brute force on tiny inputs, invariants and the
independent formulations (literal loop / counting sort / C).  The reference's
own tests hold no numeric fixtures for this path, so these checks are what
fixes the oracle.  A dropped term, wrong sign, swapped gate/up half or
transposed weight fails at least one test here.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import c_oracle
from oracle import sparse_layer_oracle as O


def g(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------ RMSNorm
def test_rmsnorm_closed_form_f64():
    x = torch.randn(7, 96, generator=g(0))
    w = 1 + 0.1 * torch.randn(96, generator=g(1))
    xd = x.double().numpy()
    ref = xd / np.sqrt((xd ** 2).mean(-1, keepdims=True) + 1e-6) * w.double().numpy()
    got = O.rmsnorm(x, w, 1e-6).double().numpy()
    assert np.max(np.abs(got - ref)) <= 1e-5 * np.max(np.abs(ref))


def test_rmsnorm_unit_rms_and_library():
    x = torch.randn(5, 3, 128, generator=g(2)) * 3.0
    y = O.rmsnorm(x, None, 1e-6)
    assert torch.allclose(y.pow(2).mean(-1).sqrt(), torch.ones(5, 3), atol=1e-5)
    w = torch.rand(128, generator=g(3)) + 0.5
    assert torch.allclose(O.rmsnorm(x, w, 1e-6), F.rms_norm(x, (128,), w, 1e-6), rtol=1e-5, atol=1e-6)


def test_rmsnorm_extreme_scales_and_dtype():
    # the reference's own stability test (Src/tests/test_model.py:31-43)
    for s in (1e-6, 1e6):
        y = O.rmsnorm(torch.randn(2, 10, 128, generator=g(4)) * s, torch.ones(128))
        assert torch.isfinite(y).all()
    xb = torch.randn(4, 64, generator=g(5)).bfloat16()
    assert O.rmsnorm(xb, torch.ones(64)).dtype == torch.bfloat16


def test_rmsnorm_scale_equivariance():
    x = torch.randn(3, 256, generator=g(6))
    assert torch.allclose(O.rmsnorm(x, None), O.rmsnorm(x * 37.0, None), rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------ RoPE table
def test_rope_table_closed_form():
    L, D, theta = 300, 64, 10000.0
    cos, sin = O.rope_table(L, D, theta)
    assert cos.shape == (L, D) and cos.dtype == torch.float32
    for pos in (0, 1, 2, 17, 299):
        for d in (0, 1, 5, 31):
            ang = float(np.float32(pos)) * (1.0 / theta ** (2 * d / D))
            for half in (0, D // 2):
                assert abs(cos[pos, d + half].item() - math.cos(ang)) <= 2e-7
                assert abs(sin[pos, d + half].item() - math.sin(ang)) <= 2e-7
    assert torch.all(cos[0] == 1) and torch.all(sin[0] == 0)
    # d = 0 has unit frequency: angle == position
    assert abs(sin[7, 0].item() - math.sin(7.0)) <= 2e-7


def test_rope_table_scaling_factor():
    c1, s1 = O.rope_table(64, 32, 10000.0, scaling_factor=2.0)
    c2, s2 = O.rope_table(32, 32, 10000.0)
    assert torch.allclose(c1[::2], c2, atol=1e-6) and torch.allclose(s1[::2], s2, atol=1e-6)


# ------------------------------------------------------------------ RoPE apply
def _rot_closed_form(x, cos, sin):
    B, Hh, L, D = x.shape
    out = np.zeros((B, Hh, L, D))
    xd = x.double().numpy()
    c = cos.double().numpy()
    s = sin.double().numpy()
    for l in range(L):
        for d in range(D // 2):
            a, b = xd[:, :, l, d], xd[:, :, l, d + D // 2]
            out[:, :, l, d] = a * c[l, d] - b * s[l, d]
            out[:, :, l, d + D // 2] = a * s[l, d] + b * c[l, d]
    return out


def test_rope_apply_closed_form_and_gqa():
    B, Hq, Hkv, L, D = 2, 4, 2, 9, 16
    q = torch.randn(B, Hq, L, D, generator=g(7))
    k = torch.randn(B, Hkv, L, D, generator=g(8))
    cos, sin = O.rope_table(L, D)
    qr, kr = O.rope_apply(q, k, cos, sin)
    assert np.max(np.abs(qr.double().numpy() - _rot_closed_form(q, cos, sin))) < 1e-6
    assert np.max(np.abs(kr.double().numpy() - _rot_closed_form(k, cos, sin))) < 1e-6
    # k is independent of the number of query heads
    _, kr2 = O.rope_apply(q[:, :1], k, cos, sin)
    assert torch.equal(kr, kr2)


def test_rope_invariants():
    B, Hh, L, D = 1, 2, 33, 32
    q = torch.randn(B, Hh, L, D, generator=g(9))
    k = torch.randn(B, Hh, L, D, generator=g(10))
    cos, sin = O.rope_table(L, D)
    qr, kr = O.rope_apply(q, k, cos, sin)
    # per-pair norm preservation (the reference's own smoke check, cuda_opt_wrapper.py:537-538)
    def pair_norm(x):
        return x[..., : D // 2] ** 2 + x[..., D // 2:] ** 2
    assert torch.allclose(pair_norm(q), pair_norm(qr), rtol=1e-5, atol=1e-5)
    # inverse rotation
    qb, _ = O.rope_apply(qr, kr, cos, -sin)
    assert torch.allclose(qb, q, atol=1e-5)
    # relative-position property: <R(m)q, R(n)k> = <R(m-n)q, k>
    qv, kv = q[0, 0, 0], k[0, 0, 0]
    qs = qv.expand(1, 1, L, D).contiguous()
    ks = kv.expand(1, 1, L, D).contiguous()
    qall, kall = O.rope_apply(qs, ks, cos, sin)
    m, n = 20, 7
    lhs = (qall[0, 0, m] * kall[0, 0, n]).sum()
    rhs = (qall[0, 0, m - n] * kv).sum()
    assert abs(lhs.item() - rhs.item()) < 1e-4


def test_fused_rope_matches_full_table_form():
    B, Hq, Hkv, L, D = 1, 2, 1, 6, 8
    q = torch.randn(B, Hq, L, D, generator=g(11))
    k = torch.randn(B, Hkv, L, D, generator=g(12))
    ch, sh = O.fused_rope_table(32, D)
    off = 5
    qf, kf = O.fused_rope_apply(q, k, ch, sh, off)
    cos = torch.cat([ch, ch], -1)[off:off + L]
    sin = torch.cat([sh, sh], -1)[off:off + L]
    qr, kr = O.rope_apply(q, k, cos, sin)
    assert torch.equal(qf, qr) and torch.equal(kf, kr)
    # half table agrees with the float64-derived one to float32 trig accuracy at small angles
    c64, s64 = O.rope_table(32, D)
    assert torch.allclose(ch, c64[:, : D // 2], atol=1e-5)


def test_fused_rope_table_both_halves_closed_form():
    """cos AND sin of the half-width float32 table against math.cos / math.sin of pos * theta^(-d/half);
    a negated or swapped sin half fails here (sin(1) > 0 at position 1, frequency 1)."""
    D, theta, L = 16, 10000.0, 40
    ch, sh = O.fused_rope_table(L, D, theta)
    half = D // 2
    assert ch.shape == (L, half) and sh.shape == (L, half) and ch.dtype == torch.float32
    for pos in (0, 1, 2, 5, 17, 39):
        for d in range(half):
            ang = pos * theta ** (-d / half)
            # float32 frequency and product rounding: relative 2^-23 each on an angle of up to 39
            tol = 3e-7 + 2.5e-7 * abs(ang)
            assert abs(ch[pos, d].item() - math.cos(ang)) <= tol, (pos, d)
            assert abs(sh[pos, d].item() - math.sin(ang)) <= tol, (pos, d)
    assert torch.all(ch[0] == 1) and torch.all(sh[0] == 0)
    assert abs(sh[1, 0].item() - math.sin(1.0)) <= 1e-7 and sh[1, 0].item() > 0.8
    assert abs(ch[1, 0].item() - math.cos(1.0)) <= 1e-7
    # and against the float64-derived full table, both halves of it
    c64, s64 = O.rope_table(L, D, theta)
    assert torch.allclose(ch, c64[:, :half], atol=1e-5) and torch.allclose(ch, c64[:, half:], atol=1e-5)
    assert torch.allclose(sh, s64[:, :half], atol=1e-5) and torch.allclose(sh, s64[:, half:], atol=1e-5)


def test_fused_rope_apply_rotation_closed_form():
    """The fused form rotates pair (d, d + D/2) of position p + offset by +angle: checked per element
    in float64 with an offset, so the sign of the sin half is fixed independently of the table."""
    B, Hq, Hkv, L, D, off, theta = 1, 2, 1, 5, 8, 3, 10000.0
    q = torch.randn(B, Hq, L, D, generator=g(111))
    k = torch.randn(B, Hkv, L, D, generator=g(112))
    ch, sh = O.fused_rope_table(16, D, theta)
    qf, kf = O.fused_rope_apply(q, k, ch, sh, off)
    half = D // 2
    for x, y in ((q, qf), (k, kf)):
        for h in range(x.shape[1]):
            for p in range(L):
                for d in range(half):
                    ang = (p + off) * theta ** (-d / half)
                    a, b = x[0, h, p, d].item(), x[0, h, p, d + half].item()
                    assert abs(y[0, h, p, d].item() - (a * math.cos(ang) - b * math.sin(ang))) <= 2e-6
                    assert abs(y[0, h, p, d + half].item() - (a * math.sin(ang) + b * math.cos(ang))) <= 2e-6


def test_rope_bf16_single_rounding():
    q = torch.randn(1, 2, 4, 8, generator=g(13)).bfloat16()
    k = torch.randn(1, 1, 4, 8, generator=g(14)).bfloat16()
    cos, sin = O.rope_table(4, 8)
    qr, kr = O.rope_apply(q, k, cos, sin)
    assert qr.dtype == torch.bfloat16
    q32, _ = O.rope_apply(q.float(), k.float(), cos, sin)
    assert torch.equal(qr, q32.bfloat16())


# ------------------------------------------------------------------ router + routing
def test_router_logits_f64():
    x = torch.randn(33, 40, generator=g(15))
    w = torch.randn(6, 40, generator=g(16)) * 0.02
    ref = x.double() @ w.double().T
    assert torch.allclose(O.router_logits(x, w).double(), ref, rtol=1e-5, atol=1e-7)


def _brute_topk(vals, k):
    # full descending sort, lower index first among equals
    order = sorted(range(len(vals)), key=lambda i: (-vals[i], i))
    return order[:k]


@pytest.mark.parametrize("E,k", [(4, 1), (4, 2), (8, 2), (8, 3), (64, 6)])
def test_routing_brute_force(E, k):
    logits = torch.randn(50, E, generator=g(17 + E + k))
    for temp in (1.0, 0.7):
        i1, w1 = O.route_softmax_topk_renorm(logits, k, temp)
        i2, w2 = O.route_topk_softmax(logits, k, temp)
        assert torch.equal(i1, i2)
        for t in range(50):
            row = (logits[t].double() / temp)
            assert i1[t].tolist() == _brute_topk(row.tolist(), k)
            p = torch.softmax(row, -1)
            sel = p[i1[t]]
            assert torch.allclose(w1[t].double(), sel / sel.sum(), atol=1e-6)
            assert torch.allclose(w2[t].double(), torch.softmax(row[i2[t]], -1), atol=1e-6)
        assert torch.allclose(w1.sum(-1), torch.ones(50), atol=1e-5)
        assert torch.allclose(w2.sum(-1), torch.ones(50), atol=1e-5)
        assert torch.allclose(w1, w2, atol=1e-6)
        assert i1.dtype == torch.int64


def test_capacity_known_values():
    assert O.capacity(512, 2, 8, 1.25) == 160
    assert O.capacity(64, 2, 8, 1.25) == 20
    assert O.capacity(16384, 2, 8, 1.25) == 5120
    assert O.capacity(4096, 6, 64, 1.5) == 576
    assert O.capacity(512, 2, 8, 1.1) == 140      # 140.8 truncates; 128*1.1 is not 141
    assert O.capacity(7, 2, 4, 1.25) == 4


# ------------------------------------------------------------------ dispatch
@pytest.mark.parametrize("T,E,k,C", [(16, 4, 2, 5), (16, 8, 3, 4), (9, 4, 1, 100), (12, 4, 2, 0),
                                     (40, 8, 2, 10), (64, 64, 6, 9)])
def test_dispatch_three_formulations(T, E, k, C):
    gen = g(100 + T + E + k + C)
    logits = torch.randn(T, E, generator=gen)
    idx = torch.topk(logits, k, -1)[1]
    x = torch.randn(T, 6, generator=gen)
    ei_l, tm_l = O.dispatch_loop(x, idx, E, C)
    ei_v, tm_v = O.dispatch_vectorized(x, idx, E, C)
    tm_c, slot_c, hist_c, kept_c, dropped_c = c_oracle.fcfs_dispatch(idx.numpy(), E, C)
    assert torch.equal(tm_l, tm_v) and torch.equal(ei_l, ei_v)
    assert np.array_equal(tm_l.numpy(), tm_c)
    _, slot_v, hist_v, kept_v = O.dispatch_plan_vectorized(idx, E, C)
    assert np.array_equal(slot_v.numpy(), slot_c)
    assert np.array_equal(hist_v.numpy(), hist_c) and np.array_equal(kept_v.numpy(), kept_c)
    # invariants
    hist = torch.bincount(idx.reshape(-1), minlength=E)
    assert np.array_equal(hist.numpy(), hist_c)
    assert np.array_equal(np.minimum(hist.numpy(), C), kept_c)
    assert kept_c.sum() + dropped_c == T * k
    for e in range(E):
        row = tm_c[e]
        n = kept_c[e]
        assert (row[:n] >= 0).all() and (row[n:] == -1).all()
        assert (np.diff(row[:n]) > 0).all()
        assert all(idx.reshape(-1)[m] == e for m in row[:n])
    occ = tm_c[tm_c >= 0]
    assert len(set(occ.tolist())) == len(occ)
    # padded rows are zero, occupied rows are the source tokens
    for e in range(E):
        for pos in range(C):
            m = tm_c[e, pos]
            if m < 0:
                assert torch.all(ei_l[e, pos] == 0)
            else:
                assert torch.equal(ei_l[e, pos], x[m // k])


def test_dispatch_special_cases():
    # everything to one expert: first C assignments in order survive
    idx = torch.zeros(10, 1, dtype=torch.int64)
    tm, slot, hist, kept, dropped = c_oracle.fcfs_dispatch(idx.numpy(), 4, 3)
    assert tm[0].tolist() == [0, 1, 2] and dropped == 7 and hist[0] == 10
    assert slot.tolist() == [0, 1, 2] + [-1] * 7
    # hand-worked example, T=4, k=2, E=3, C=2
    idx = torch.tensor([[0, 1], [0, 2], [0, 1], [1, 2]])
    tm, slot, hist, kept, dropped = c_oracle.fcfs_dispatch(idx.numpy(), 3, 2)
    assert tm.tolist() == [[0, 2], [1, 5], [3, 7]]
    assert slot.tolist() == [0, 0, 1, 0, -1, 1, -1, 1]
    assert hist.tolist() == [3, 3, 2] and kept.tolist() == [2, 2, 2] and dropped == 2


# ------------------------------------------------------------------ experts
def test_swiglu_expert_f64():
    H, I = 12, 20
    x = torch.randn(5, H, generator=g(20))
    wgu = torch.randn(2 * I, H, generator=g(21)) * 0.3
    wd = torch.randn(H, I, generator=g(22)) * 0.3
    xd = x.double()
    gate = xd @ wgu[:I].double().T
    up = xd @ wgu[I:].double().T
    ref = ((gate / (1 + torch.exp(-gate))) * up) @ wd.double().T
    assert torch.allclose(O.swiglu_expert(x, wgu, wd).double(), ref, rtol=1e-5, atol=1e-6)
    # swapping the halves must change the answer (guards the gate/up convention)
    swapped = torch.cat([wgu[I:], wgu[:I]], 0)
    assert not torch.allclose(O.swiglu_expert(x, swapped, wd).double(), ref, rtol=1e-3, atol=1e-4)


# ------------------------------------------------------------------ combine + whole layer
def _tiny_layer(seed, T=24, H=16, I=24, E=4):
    gen = g(seed)
    x = torch.randn(T, H, generator=gen)
    wg = torch.randn(E, H, generator=gen) * 0.5
    wgu = [torch.randn(2 * I, H, generator=gen) * 0.2 for _ in range(E)]
    wd = [torch.randn(H, I, generator=gen) * 0.2 for _ in range(E)]
    return x, wg, wgu, wd


def test_combine_formulations_and_linearity():
    x, wg, wgu, wd = _tiny_layer(30)
    r = O.moe_forward_capacity(x, wg, wgu, wd, k=2, capacity_factor=0.75, literal_loops=True)
    assert (r["slot"] < 0).any(), "case must drop something"
    T, k = r["indices"].shape
    out_v = O.combine_vectorized(r["expert_outputs"], r["token_map"], r["weights"], T, k)
    assert torch.equal(out_v, r["out"])
    out_c = c_oracle.combine_f32(r["expert_outputs"].numpy(), r["token_map"].numpy(),
                                 r["weights"].numpy(), T, k)
    assert np.array_equal(out_c, r["out"].numpy())
    out2 = O.combine_loop(r["expert_outputs"], r["token_map"], 2.0 * r["weights"], T, k)
    assert torch.allclose(out2, 2.0 * r["out"], rtol=1e-6, atol=1e-7)
    # brute force: sum over kept assignments
    bf = torch.zeros_like(r["out"]).double()
    for a in range(T * k):
        s = r["slot"][a].item()
        if s >= 0:
            e = r["indices"].reshape(-1)[a].item()
            bf[a // k] += r["weights"].reshape(-1)[a].double() * r["expert_outputs"][e, s].double()
    assert torch.allclose(r["out"].double(), bf, rtol=1e-5, atol=1e-6)
    # fully dropped tokens stay zero; weights not renormalised
    for t in range(T):
        if (r["slot"][t * k:(t + 1) * k] < 0).all():
            assert torch.all(r["out"][t] == 0)


def test_capacity_layer_equals_nocap_when_nothing_dropped():
    x, wg, wgu, wd = _tiny_layer(31)
    a = O.moe_forward_capacity(x, wg, wgu, wd, k=2, capacity_factor=100.0, literal_loops=True)
    b = O.moe_forward_nocap(x, wg, wgu, wd, k=2)
    assert torch.equal(a["indices"], b["indices"])
    assert (a["slot"] >= 0).all()
    assert torch.allclose(a["out"], b["out"], rtol=1e-5, atol=1e-6)
    assert torch.equal(a["aux"], b["aux"])


def test_nocap_dense_brute_force():
    x, wg, wgu, wd = _tiny_layer(32)
    r = O.moe_forward_nocap(x.view(2, 12, 16), wg, wgu, wd, k=2)
    assert r["out"].shape == (2, 12, 16)
    dense = torch.zeros(24, 16, dtype=torch.float64)
    for e in range(4):
        y = O.swiglu_expert(x, wgu[e], wd[e]).double()
        wsel = ((r["indices"] == e).double() * r["weights"].double()).sum(-1, keepdim=True)
        dense += wsel * y
    assert torch.allclose(r["out"].reshape(24, 16).double(), dense, rtol=1e-5, atol=1e-6)


def test_aux_loss_uniform_and_closed_form():
    E, T, k = 8, 64, 2
    logits = torch.zeros(T, E)                       # uniform importance 1/E
    idx = torch.stack([torch.arange(T) % E, (torch.arange(T) + 1) % E], -1)   # uniform usage
    assert abs(O.aux_loss(logits, idx, E, 0.01).item() - 0.01) < 1e-8
    logits = torch.randn(T, E, generator=g(33))
    idx = torch.topk(logits, k, -1)[1]
    usage = torch.bincount(idx.reshape(-1), minlength=E).double() / (T * k)
    imp = torch.softmax(logits.double(), -1).mean(0)
    ref = min(float((usage * imp).sum() * E * 0.01), 1.0)
    assert abs(O.aux_loss(logits, idx, E, 0.01).item() - ref) < 1e-7
    assert O.aux_loss(logits, idx, E, 1e6).item() == 1.0     # clamp


def test_temperature_changes_weights_not_indices():
    x, wg, wgu, wd = _tiny_layer(34)
    a = O.moe_forward_capacity(x, wg, wgu, wd, k=2, temperature=1.0)
    b = O.moe_forward_capacity(x, wg, wgu, wd, k=2, temperature=2.0)
    assert torch.equal(a["indices"], b["indices"])
    assert not torch.allclose(a["weights"], b["weights"])


# ------------------------------------------------------------------ MoD
def test_mod_router_probs_closed_form_f64():
    """sigmoid((x.w + b) / T) written out in float64 with bias != 0 and temperature != 1: a dropped
    bias, a temperature that multiplies or sits outside the sigmoid, or a transposed weight fails."""
    gen = g(135)
    B, L, H = 2, 9, 24
    x = torch.randn(B, L, H, generator=gen)
    w = torch.randn(1, H, generator=gen) * 0.3
    for b, T in ((0.0, 1.0), (0.7, 1.0), (-0.4, 2.5), (1.3, 0.5)):
        bias = torch.tensor([b])
        p = O.mod_router_probs(x, w, bias, T)
        assert p.shape == (B, L, 1) and p.dtype == torch.float32
        xd, wd = x.double().numpy(), w.double().numpy()[0]
        for bi in range(B):
            for li in range(L):
                z = (float(np.dot(xd[bi, li], wd)) + b) / T
                assert abs(p[bi, li, 0].item() - 1.0 / (1.0 + math.exp(-z))) <= 2e-7
    # no bias at all == zero bias
    assert torch.equal(O.mod_router_probs(x, w, None, 1.7), O.mod_router_probs(x, w, torch.zeros(1), 1.7))


def test_mod_router_probs_special_cases():
    x = torch.randn(3, 4, 8, generator=g(136))
    # w = 0: every token gets sigmoid(b / T)
    for b, T in ((0.9, 3.0), (-2.0, 0.25)):
        p = O.mod_router_probs(x, torch.zeros(1, 8), torch.tensor([b]), T)
        assert torch.allclose(p, torch.full_like(p, 1.0 / (1.0 + math.exp(-b / T))), atol=1e-7)
    # w = 0, b = 0: exactly one half
    assert torch.all(O.mod_router_probs(x, torch.zeros(1, 8), None, 1.0) == 0.5)
    # monotone in the bias, antisymmetric in the sign of the input: p(x) + p(-x) = 1 without bias
    w = torch.randn(1, 8, generator=g(137))
    assert torch.allclose(O.mod_router_probs(x, w, None, 2.0) + O.mod_router_probs(-x, w, None, 2.0),
                          torch.ones(3, 4, 1), atol=1e-6)
    assert torch.all(O.mod_router_probs(x, w, torch.tensor([1.0]), 2.0) > O.mod_router_probs(x, w, None, 2.0))
    # a larger temperature pulls every probability toward one half
    far = (O.mod_router_probs(x, w, None, 1.0) - 0.5).abs()
    near = (O.mod_router_probs(x, w, None, 4.0) - 0.5).abs()
    assert torch.all(near <= far)


def test_mod_router_train_mask_ste_gradient_and_aux():
    """Training branch of the MoD router: the mask is the brute-force ranking with exactly int(N*cf) ones; the
    routing weights have the mask's value (to one ulp of the float32 (m - p) + p) and the gradient of the
    probabilities, p(1-p)/T per logit in float64 terms; the auxiliary loss is (k/N - cf)^2 and a constant."""
    gen = g(141)
    B, L, H = 3, 11, 20
    x = torch.randn(B, L, H, generator=gen)
    for cf, b, T in ((0.5, 0.3, 1.0), (0.125, -0.2, 2.0), (0.9, 0.0, 0.7)):
        w = (torch.randn(1, H, generator=gen) * 0.4).requires_grad_()
        bias = torch.tensor([b], requires_grad=True)
        xg = x.clone().requires_grad_()
        weights, probs, mask, aux = O.mod_router_train(xg, w, bias, T, cf)
        n, k = B * L, int(B * L * cf)
        assert weights.shape == probs.shape == mask.shape == (B, L, 1)
        pd = 1.0 / (1.0 + np.exp(-((x.double().numpy() @ w.detach().double().numpy()[0]) + b) / T))   # [B, L]
        order = sorted(range(n), key=lambda i: -pd.reshape(-1)[i])
        want = np.zeros(n)
        want[order[:k]] = 1.0
        assert int(mask.sum()) == k and np.array_equal(mask.reshape(-1).numpy(), want)
        assert (weights.detach() - mask).abs().max().item() <= 1.2e-7
        assert not mask.requires_grad and not aux.requires_grad
        assert abs(aux.item() - (k / n - cf) ** 2) <= 1e-7
        # a cotangent that differs per token: a gradient that ignored it, or used the mask's, would fail
        cot = torch.randn(B, L, 1, generator=gen)
        weights.backward(cot)
        gl = cot.double().numpy()[..., 0] * pd * (1.0 - pd) / T                       # d loss / d logit
        assert np.allclose(bias.grad.double().numpy(), gl.sum(), atol=1e-5)
        assert np.allclose(w.grad.double().numpy()[0], np.einsum("bl,blh->h", gl, x.double().numpy()), atol=1e-5)
        assert np.allclose(xg.grad.double().numpy(), gl[..., None] * w.detach().double().numpy()[0], atol=1e-6)
    # capacity_factor of one or more: every token is computed
    weights, _, mask, aux = O.mod_router_train(x, torch.randn(1, H, generator=gen), None, 1.0, 1.0)
    assert mask.all() and abs(aux.item()) <= 1e-12


def test_mod_moe_block_scores_and_selection_f64():
    """The block's scores are x.w + b in float64 terms and its selection is the brute-force top-keep of them."""
    gen = g(138)
    B, L, H, I, E, keep = 2, 12, 16, 24, 4, 3
    x = torch.randn(B, L, H, generator=gen)
    wm = torch.randn(1, H, generator=gen)
    bm = torch.tensor([0.25])
    _, wg, wgu, wd = _tiny_layer(139, H=H, I=I, E=E)
    r = O.mod_moe_block(x, wm, bm, keep, dict(gate_weight=wg, gate_up_weights=wgu, down_weights=wd,
                                              k=2, capacity_factor=1.5))
    ref = (x.double() @ wm.double().T).squeeze(-1) + 0.25
    assert torch.allclose(r["scores"].double(), ref, atol=1e-5)
    for b in range(B):
        order = sorted(range(L), key=lambda i: (-ref[b, i].item(), i))[:keep]
        assert r["selected"][b].tolist() == sorted(order)


def test_mod_eval_mask_threshold():
    p = torch.rand(2, 16, 1, generator=g(35))
    mask = O.mod_router_eval_mask(p, 0.5)
    n, cap = 32, 16
    srt = sorted(p.flatten().tolist())
    thr = srt[max(1, n - cap) - 1]
    assert mask.flatten().tolist() == [1.0 if v >= thr else 0.0 for v in p.flatten().tolist()]
    assert int(mask.sum()) == cap + 1        # the reference's off-by-one


def test_mod_select_per_sequence():
    s = torch.randn(3, 40, generator=g(36))
    sel = O.mod_select_per_sequence(s, 5)
    for b in range(3):
        order = sorted(range(40), key=lambda i: (-s[b, i].item(), i))[:5]
        assert sel[b].tolist() == sorted(order)
    # ties go to the lower position
    assert O.mod_select_per_sequence(torch.tensor([[1.0, 2.0, 2.0, 2.0]]), 2).tolist() == [[1, 2]]


def test_mod_moe_block_skip_tokens_untouched():
    gen = g(37)
    B, L, H, I, E = 2, 16, 16, 24, 4
    x = torch.randn(B, L, H, generator=gen)
    wm = torch.randn(1, H, generator=gen)
    _, wg, wgu, wd = _tiny_layer(38, H=H, I=I, E=E)
    r = O.mod_moe_block(x, wm, None, 4, dict(gate_weight=wg, gate_up_weights=wgu, down_weights=wd,
                                             k=2, capacity_factor=1.5))
    keep = torch.zeros(B, L, dtype=torch.bool)
    keep.scatter_(1, r["selected"], True)
    assert torch.equal(r["block_out"][~keep], x[~keep])
    assert torch.allclose(r["block_out"][keep] - x[keep], r["out"].reshape(-1, H), atol=1e-6)


# --------------------------------------------------------------------------- backward restatements
def test_rmsnorm_backward_matches_autograd_and_gradcheck():
    g = torch.Generator().manual_seed(31)
    x = torch.randn(7, 24, generator=g, dtype=torch.float64)
    w = torch.randn(24, generator=g, dtype=torch.float64) * 0.3 + 1.0
    dy = torch.randn(7, 24, generator=g, dtype=torch.float64)

    def f64(xx, ww):     # float64 closed form of the forward (O.rmsnorm up-casts to float32 only)
        return xx * torch.rsqrt(xx.pow(2).mean(-1, keepdim=True) + 1e-6) * ww

    xr, wr = x.clone().requires_grad_(), w.clone().requires_grad_()
    gx, gw = torch.autograd.grad((f64(xr, wr) * dy).sum(), [xr, wr])
    dx, dw = O.rmsnorm_backward(x.float(), w.float(), dy.float())
    assert torch.allclose(dx.double(), gx, rtol=2e-5, atol=2e-6)
    assert torch.allclose(dw.double(), gw, rtol=2e-5, atol=2e-5)
    assert torch.autograd.gradcheck(f64, (xr, wr), eps=1e-6, atol=1e-6)
    # no weight: same formula with w = 1, dw is None
    dx1, dw1 = O.rmsnorm_backward(x.float(), None, dy.float())
    gx1, = torch.autograd.grad((f64(xr, torch.ones_like(w)) * dy).sum(), [xr])
    assert dw1 is None and torch.allclose(dx1.double(), gx1, rtol=2e-5, atol=2e-6)


def test_rope_backward_is_transpose_of_forward():
    g = torch.Generator().manual_seed(32)
    B, Hq, Hkv, L, D = 2, 3, 1, 9, 8
    cos, sin = O.fused_rope_table(32, D)
    q = torch.randn(B, Hq, L, D, generator=g).requires_grad_()
    k = torch.randn(B, Hkv, L, D, generator=g).requires_grad_()
    dq_o, dk_o = torch.randn(B, Hq, L, D, generator=g), torch.randn(B, Hkv, L, D, generator=g)
    qo, ko = O.fused_rope_apply(q, k, cos, sin, position_offset=5)
    gq, gk = torch.autograd.grad((qo * dq_o).sum() + (ko * dk_o).sum(), [q, k])
    dq, dk = O.rope_backward(dq_o, dk_o, cos, sin, position_offset=5)
    assert torch.allclose(dq, gq, rtol=1e-6, atol=1e-6) and torch.allclose(dk, gk, rtol=1e-6, atol=1e-6)
    # rotating forward and then with the inverse returns the input
    back_q, back_k = O.rope_backward(qo.detach(), ko.detach(), cos, sin, position_offset=5)
    assert torch.allclose(back_q, q.detach(), atol=1e-5) and torch.allclose(back_k, k.detach(), atol=1e-5)


def test_swiglu_backward_matches_autograd():
    g = torch.Generator().manual_seed(33)
    gate = torch.randn(5, 12, generator=g, dtype=torch.float64).requires_grad_()
    up = (torch.randn(5, 12, generator=g, dtype=torch.float64) * 2).requires_grad_()
    dout = torch.randn(5, 12, generator=g, dtype=torch.float64)
    f = lambda a, b: a * torch.nn.functional.silu(b)
    gg, gu = torch.autograd.grad((f(gate, up) * dout).sum(), [gate, up])
    dg, du = O.swiglu_backward(gate.detach().float(), up.detach().float(), dout.float())
    assert torch.allclose(dg.double(), gg, rtol=1e-5, atol=1e-6) and torch.allclose(du.double(), gu, rtol=1e-5, atol=1e-6)
    assert torch.autograd.gradcheck(f, (gate, up), eps=1e-6, atol=1e-6)


def test_layer_grads_gradcheck_fixed_routing():
    """The layer's gradient oracle is autograd over the forward restatement; with the discrete routing
    held fixed the forward is smooth, so float64 finite differences must agree with it."""
    g = torch.Generator().manual_seed(34)
    T, H, E, I, k = 6, 8, 3, 5, 2
    x = torch.randn(T, H, generator=g, dtype=torch.float64).requires_grad_()
    wg = (torch.randn(E, H, generator=g, dtype=torch.float64) * 0.5).requires_grad_()
    wgu = (torch.randn(E, 2 * I, H, generator=g, dtype=torch.float64) * 0.3).requires_grad_()
    wd = (torch.randn(E, H, I, generator=g, dtype=torch.float64) * 0.3).requires_grad_()
    idx = torch.topk(torch.softmax(x.detach() @ wg.detach().T, -1), k, dim=-1).indices

    def f(xx, wgg, wguu, wdd):
        probs = torch.softmax(xx @ wgg.T, -1)
        top = probs.gather(1, idx)
        w = top / (top.sum(-1, keepdim=True) + 1e-9)
        out = torch.zeros_like(xx)
        for e in range(E):
            for j in range(k):
                m = idx[:, j] == e
                gu = xx[m] @ wguu[e].T
                h = torch.nn.functional.silu(gu[:, :I]) * gu[:, I:]
                out[m] = out[m] + (h @ wdd[e].T) * w[m, j:j + 1]
        return out

    # the double-precision closed form equals the float32 oracle forward ...
    ref = O.moe_forward_nocap(x.detach().float(), wg.detach().float(), [w_.float() for w_ in wgu.detach()],
                              [w_.float() for w_ in wd.detach()], k)
    assert torch.equal(ref["indices"], idx)
    assert torch.allclose(ref["out"].double(), f(x, wg, wgu, wd).detach(), rtol=1e-4, atol=1e-5)
    # ... and its autograd gradient passes the finite-difference check
    assert torch.autograd.gradcheck(f, (x, wg, wgu, wd), eps=1e-6, atol=1e-5)
    # layer_grads (autograd over the float32 oracle) agrees with autograd over the closed form
    cot = torch.randn(T, H, generator=g, dtype=torch.float64)
    g64 = torch.autograd.grad((f(x, wg, wgu, wd) * cot).sum(), [x, wg, wgu, wd])
    got = O.layer_grads(lambda xx, wgg, *ws: O.moe_forward_nocap(xx, wgg, list(ws[:E]), list(ws[E:]), k)["out"],
                        [x, wg] + list(wgu.detach()) + list(wd.detach()), [cot])
    assert torch.allclose(got[0].double(), g64[0], rtol=1e-3, atol=1e-5)
    assert torch.allclose(got[1].double(), g64[1], rtol=1e-3, atol=1e-5)
    assert torch.allclose(torch.stack(got[2:2 + E]).double(), g64[2], rtol=1e-3, atol=1e-5)
    assert torch.allclose(torch.stack(got[2 + E:]).double(), g64[3], rtol=1e-3, atol=1e-5)


# --------------------------------------------------------------------------- training-step ops
def test_fused_loss_closed_form_and_masking():
    g = torch.Generator().manual_seed(61)
    T, V = 40, 37
    z = torch.randn(T, V, generator=g, dtype=torch.float64) * 3
    y = torch.randint(0, V, (T,), generator=g)
    y[3] = -100
    y[7] = V + 5            # out of range: ignored like the pad id
    y[11] = -1
    r = O.fused_loss(z.float(), y)
    keep = torch.tensor([i for i in range(T) if i not in (3, 7, 11)])
    lse = torch.logsumexp(z[keep], -1)
    ref = (lse - z[keep, y[keep]]).mean()
    assert abs(r["loss"].item() - ref.item()) < 1e-5 and r["valid_tokens"].item() == T - 3
    assert abs(r["accuracy"].item() - (z[keep].argmax(-1) == y[keep]).double().mean().item()) < 1e-6
    assert abs(r["perplexity"].item() - min(math.exp(ref.item()), math.exp(15.0))) / r["perplexity"].item() < 1e-4
    # uniform logits: loss = log V exactly, accuracy = share of label 0 (first index wins the arg-max)
    u = O.fused_loss(torch.zeros(T, V), y)
    assert abs(u["loss"].item() - math.log(V)) < 1e-6
    # weights: weighted mean over valid tokens
    w = torch.rand(T, generator=g)
    rw = O.fused_loss(z.float(), y, loss_weights=w)
    refw = ((lse - z[keep, y[keep]]) * w[keep].double()).sum() / w[keep].double().sum()
    assert abs(rw["loss"].item() - refw.item()) < 1e-5
    # all tokens ignored
    e = O.fused_loss(z.float(), torch.full((T,), -100))
    assert e["loss"].item() == 0.0 and e["valid_tokens"].item() == 0 and math.isinf(e["perplexity"].item())


def test_clip_grad_norm_closed_form():
    g = torch.Generator().manual_seed(62)
    grads = [torch.randn(5, 7, generator=g), torch.randn(11, generator=g) * 3, torch.randn(2, 3, 4, generator=g)]
    total = math.sqrt(sum(float((x.double() ** 2).sum()) for x in grads))
    n, clipped = O.clip_grad_norm(grads, max_norm=1.0)
    assert abs(n.item() - total) < 1e-5
    new_total = math.sqrt(sum(float((x.double() ** 2).sum()) for x in clipped))
    assert abs(new_total - 1.0) < 1e-4
    n2, same = O.clip_grad_norm(grads, max_norm=1e6)
    assert all(torch.equal(a, b) for a, b in zip(grads, same))
    params = [torch.nn.Parameter(torch.zeros_like(x)) for x in grads]
    for p_, x in zip(params, grads):
        p_.grad = x.clone()
    lib_norm = torch.nn.utils.clip_grad_norm_(params, 1.0)
    assert abs(lib_norm.item() - n.item()) < 1e-5
    assert all(torch.allclose(p_.grad, c, atol=1e-6) for p_, c in zip(params, clipped))


# --------------------------------------------------------------------------- attention
def test_attention_standard_brute_force_and_sdpa():
    g = torch.Generator().manual_seed(81)
    B, H, L, D = 2, 3, 11, 8
    q = torch.randn(B, H, L, D, generator=g)
    k = torch.randn(B, H, L, D, generator=g)
    v = torch.randn(B, H, L, D, generator=g)
    scale = D ** -0.5
    out = O.attention_standard(q, k, v, scale)
    ref = torch.zeros(B, L, H, D, dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            for i in range(L):
                s = torch.tensor([float(q[b, h, i].double() @ k[b, h, j].double()) * scale for j in range(i + 1)],
                                 dtype=torch.float64)
                p = torch.exp(s - s.max())
                p = p / p.sum()
                ref[b, i, h] = (p.unsqueeze(1) * v[b, h, :i + 1].double()).sum(0)
    assert torch.allclose(out.double(), ref.reshape(B, L, H * D), atol=1e-5)
    sdpa = F.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=True)
    assert torch.allclose(out.double(), sdpa.transpose(1, 2).reshape(B, L, H * D), atol=1e-5)
    # the first query attends to the first key only
    assert torch.allclose(out.view(B, L, H, D)[:, 0], v[:, :, 0].transpose(0, 1).transpose(0, 1), atol=1e-6)


def test_attention_standard_with_cached_keys():
    """Keys in front of the queries: the last L rows of a full-length call, one new token seeing every key
    (the only cached case the reference's own mask admits), and a brute-force sum."""
    g = torch.Generator().manual_seed(83)
    B, H, Lk, D = 2, 2, 13, 8
    q = torch.randn(B, H, Lk, D, generator=g)
    k = torch.randn(B, H, Lk, D, generator=g)
    v = torch.randn(B, H, Lk, D, generator=g)
    scale = D ** -0.5
    full = O.attention_standard(q, k, v, scale).view(B, Lk, H, D)
    for L in (1, 4, 12):
        part = O.attention_standard(q[:, :, Lk - L:], k, v, scale).view(B, L, H, D)
        assert torch.allclose(part, full[:, Lk - L:], atol=1e-6)
    one = O.attention_standard(q[:, :, -1:], k, v, scale).view(B, H, D)
    p = torch.softmax(torch.einsum("bhd,bhjd->bhj", q[:, :, -1].double(), k.double()) * scale, -1)
    assert torch.allclose(one.double(), torch.einsum("bhj,bhjd->bhd", p, v.double()), atol=1e-5)


def test_attention_standard_padding_mask():
    """A [B, Lk] mask of real (1) and padded (0) keys: with right padding every query sees a real key, and
    the result equals attention over the real keys alone (the padded ones get exp(-1e4) = 0 weight);
    an all-ones mask changes nothing; a brute-force sum with the additive -1e4 covers left padding."""
    g = torch.Generator().manual_seed(85)
    B, H, L, D = 2, 2, 12, 8
    q = torch.randn(B, H, L, D, generator=g)
    k = torch.randn(B, H, L, D, generator=g)
    v = torch.randn(B, H, L, D, generator=g)
    scale = D ** -0.5
    assert torch.equal(O.attention_standard(q, k, v, scale, torch.ones(B, L)), O.attention_standard(q, k, v, scale))
    real = [9, 5]
    mask = torch.zeros(B, L)
    for b, n in enumerate(real):
        mask[b, :n] = 1
    out = O.attention_standard(q, k, v, scale, mask).view(B, L, H, D)
    for b, n in enumerate(real):
        head = O.attention_standard(q[b:b + 1, :, :n], k[b:b + 1, :, :n], v[b:b + 1, :, :n], scale).view(1, n, H, D)
        assert torch.allclose(out[b:b + 1, :n], head, atol=1e-6)
        # a padded query position still sees every real key and nothing else
        p = torch.softmax(torch.einsum("hid,hjd->hij", q[b, :, n:].double(), k[b, :, :n].double()) * scale, -1)
        tail = torch.einsum("hij,hjd->ihd", p, v[b, :, :n].double())
        assert torch.allclose(out[b, n:].double(), tail, atol=1e-5)
    # integer masks as a tokenizer gives them
    assert torch.equal(O.attention_standard(q, k, v, scale, mask.long()).view(B, L, H, D), out)
    # left padding, brute force in float64 with the same additive constants; query 0 sees only a padded key
    # and, like the reference, then spreads its weight over every key whose fill is -1e4 as well
    mask = torch.ones(B, L)
    mask[:, :3] = 0
    out = O.attention_standard(q, k, v, scale, mask).view(B, L, H, D)
    s = torch.einsum("bhid,bhjd->bhij", q.double(), k.double()) * scale
    s = s.masked_fill(torch.triu(torch.ones(L, L, dtype=torch.bool), 1), -1e4) + (1 - mask.double())[:, None, None, :] * -1e4
    ref = torch.einsum("bhij,bhjd->bihd", torch.softmax(s, -1), v.double())
    assert torch.allclose(out[:, 3:].double(), ref[:, 3:], atol=1e-5)
    assert torch.allclose(out[:, :3].double(), ref[:, :3], atol=2e-3)     # float32 scores near 1e4 resolve 1e-3


def test_gqa_forward_cache_round_trip():
    """use_cache returns the rotated keys and the values; feeding them back with new tokens reproduces the
    reference's quirk of rotating the new tokens at positions 0..L-1 (model.py:690-698)."""
    g = torch.Generator().manual_seed(84)
    B, L, Hd, nh, nkv = 1, 6, 16, 4, 2
    D = Hd // nh
    x = torch.randn(B, L, Hd, generator=g)
    w = [torch.randn(n, Hd, generator=g) * 0.3 for n in (nh * D, nkv * D, nkv * D, Hd)]
    out, (kc, vc) = O.gqa_forward(x, *w, nh, nkv, use_cache=True)
    assert kc.shape == (B, nkv, L, D) and vc.shape == (B, nkv, L, D)
    assert torch.equal(out, O.gqa_forward(x, *w, nh, nkv))
    x1 = torch.randn(B, 1, Hd, generator=g)
    out1, (kc1, vc1) = O.gqa_forward(x1, *w, nh, nkv, past_key_value=(kc, vc), use_cache=True)
    assert kc1.shape == (B, nkv, L + 1, D) and torch.equal(kc1[:, :, :L], kc) and torch.equal(vc1[:, :, :L], vc)
    # the new token's key is rotated at position 0, i.e. not rotated at all
    k_new = (x1 @ w[1].T).view(B, 1, nkv, D).transpose(1, 2)
    assert torch.allclose(kc1[:, :, L:], k_new, atol=1e-6)
    q_new = (x1 @ w[0].T).view(B, 1, nh, D).transpose(1, 2)
    rep = nh // nkv
    p = torch.softmax(torch.einsum("bhd,bhjd->bhj", q_new[:, :, 0].double(),
                                   kc1.repeat_interleave(rep, 1).double()) * D ** -0.5, -1)
    a = torch.einsum("bhj,bhjd->bhd", p, vc1.repeat_interleave(rep, 1).double()).reshape(B, 1, nh * D)
    assert torch.allclose(out1.double(), a @ w[3].double().T, atol=2e-5)


def test_gqa_forward_matches_per_head_composition():
    g = torch.Generator().manual_seed(82)
    B, L, Hd, nh, nkv = 2, 9, 32, 4, 2
    D = Hd // nh
    x = torch.randn(B, L, Hd, generator=g)
    wq = torch.randn(nh * D, Hd, generator=g) * 0.2
    wk = torch.randn(nkv * D, Hd, generator=g) * 0.2
    wv = torch.randn(nkv * D, Hd, generator=g) * 0.2
    wo = torch.randn(Hd, Hd, generator=g) * 0.2
    out = O.gqa_forward(x, wq, wk, wv, wo, nh, nkv)
    q = (x @ wq.T).view(B, L, nh, D).transpose(1, 2)
    k = (x @ wk.T).view(B, L, nkv, D).transpose(1, 2)
    v = (x @ wv.T).view(B, L, nkv, D).transpose(1, 2)
    cos, sin = O.rope_table(L, D)
    q, k = O.rope_apply(q, k, cos, sin)
    heads = []
    for h in range(nh):
        kv = h // (nh // nkv)           # query head h reads kv head h // group size
        a = F.scaled_dot_product_attention(q[:, h:h + 1].double(), k[:, kv:kv + 1].double(), v[:, kv:kv + 1].double(),
                                           is_causal=True)
        heads.append(a[:, 0])
    ref = torch.cat(heads, dim=-1) @ wo.double().T
    assert torch.allclose(out.double(), ref, atol=2e-5)


def test_every_oracle_function_declares_its_pin():
    """Every function of the oracle names the independent check that fixes it; none is left out."""
    import inspect
    fns = [n for n, f in inspect.getmembers(O, inspect.isfunction) if f.__module__ == O.__name__]
    assert sorted(fns) == sorted(O.PINNING), set(fns) ^ set(O.PINNING)
    assert not [n for n, why in O.PINNING.items() if "unpinned" in why]


def test_attention_standard_pair_mask_and_dropout():
    """The 4-D mask and the explicit dropout mask of the oracle's attention against a float64 sum written out
    per element (additive -1e4 constants, weights scaled by keep / (1 - p)); a 4-D mask that repeats a
    [B, Lk] mask gives the 2-D path's result; keep-all with p = 0 changes nothing; keep-all with p scales the
    output by 1 / (1 - p)."""
    g = torch.Generator().manual_seed(87)
    B, H, L, Lk, D = 2, 3, 7, 9, 8
    q = torch.randn(B, H, L, D, generator=g)
    k = torch.randn(B, H, Lk, D, generator=g)
    v = torch.randn(B, H, Lk, D, generator=g)
    scale = D ** -0.5
    mask = (torch.rand(B, 1, L, Lk, generator=g) > 0.4).float()
    i = torch.arange(L)
    mask[:, 0, i, i + Lk - L] = 1
    keep = torch.rand(B, H, L, Lk, generator=g) > 0.3
    p = 0.3
    out = O.attention_standard(q, k, v, scale, mask, dropout_keep=keep, dropout_p=p).view(B, L, H, D)
    for b in range(B):
        for h in range(H):
            for qi in range(L):
                s = []
                for j in range(Lk):
                    sc = float(q[b, h, qi].double() @ k[b, h, j].double()) * scale
                    if j > qi + Lk - L:
                        sc = -1e4
                    sc += (1.0 - float(mask[b, 0, qi, j])) * -1e4
                    s.append(sc)
                mx = max(s)
                e = [math.exp(x - mx) for x in s]
                tot = sum(e)
                acc = torch.zeros(D, dtype=torch.float64)
                for j in range(Lk):
                    if keep[b, h, qi, j]:
                        acc += (e[j] / tot / (1.0 - p)) * v[b, h, j].double()
                assert torch.allclose(out[b, qi, h].double(), acc, atol=2e-5), (b, h, qi)
    pad = torch.ones(B, Lk)
    pad[0, 2] = 0
    pad[1, 5:7] = 0
    assert torch.allclose(O.attention_standard(q, k, v, scale, pad[:, None, None, :].expand(B, 1, L, Lk)),
                          O.attention_standard(q, k, v, scale, pad), atol=1e-6)
    ones = torch.ones(B, H, L, Lk, dtype=torch.bool)
    base = O.attention_standard(q, k, v, scale)
    assert torch.equal(O.attention_standard(q, k, v, scale, dropout_keep=ones, dropout_p=0.0), base)
    assert torch.allclose(O.attention_standard(q, k, v, scale, dropout_keep=ones, dropout_p=0.5), base * 2.0, atol=1e-5)


def test_attention_dropout_keep_known_answers_and_statistics():
    """The keep / drop function: with seed 0 the (batch 0, head 0) key is 0, so element (query 0, key j) is
    decided by MurmurHash3's finaliser of j, whose published values fmix32(0) = 0, fmix32(1) = 0x514e28b7,
    fmix32(2) = 0x30f4c306 fix the outcome on both sides of each threshold; the keep rate matches 1 - p within
    4 sigma; masks of different seeds, heads and batch entries are uncorrelated; p = 0 keeps everything."""
    for p, want in [(0.31, True), (0.32, False)]:       # 0x514e28b7 / 2^32 = 0.31760
        assert bool(O.attention_dropout_keep(0, 1, 1, 1, 4, p)[0, 0, 0, 1]) == want
    for p, want in [(0.19, True), (0.20, False)]:       # 0x30f4c306 / 2^32 = 0.19123
        assert bool(O.attention_dropout_keep(0, 1, 1, 1, 4, p)[0, 0, 0, 2]) == want
    assert not bool(O.attention_dropout_keep(0, 1, 1, 1, 4, 1e-9)[0, 0, 0, 0])      # hash 0 < any threshold >= 1
    assert bool(O.attention_dropout_keep(0, 2, 3, 5, 7, 0.0).all())
    B, H, L, Lk = 2, 4, 128, 160
    n = B * H * L * Lk
    for p in (0.1, 0.5, 0.9):
        m = O.attention_dropout_keep(12345, B, H, L, Lk, p).float()
        assert abs(m.mean().item() - (1 - p)) <= 4 * math.sqrt(p * (1 - p) / n)
        per_head = m.mean(dim=(2, 3))
        assert (per_head - (1 - p)).abs().max().item() <= 5 * math.sqrt(p * (1 - p) / (L * Lk))
    a = O.attention_dropout_keep(1, B, H, L, Lk, 0.5).float() - 0.5
    b = O.attention_dropout_keep(2, B, H, L, Lk, 0.5).float() - 0.5
    bound = 5 * 0.25 / math.sqrt(L * Lk)
    assert abs((a * b).mean().item()) <= 5 * 0.25 / math.sqrt(n)
    assert abs((a[0, 0] * a[0, 1]).mean().item()) <= bound and abs((a[0, 0] * a[1, 0]).mean().item()) <= bound
    # neighbouring keys and neighbouring queries of one head
    assert abs((a[..., :-1] * a[..., 1:]).mean().item()) <= 5 * 0.25 / math.sqrt(n)
    assert abs((a[:, :, :-1] * a[:, :, 1:]).mean().item()) <= 5 * 0.25 / math.sqrt(n)
    assert torch.equal(O.attention_dropout_keep(1, B, H, L, Lk, 0.5), O.attention_dropout_keep(1, B, H, L, Lk, 0.5))
