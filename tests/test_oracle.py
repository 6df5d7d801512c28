"""Pins every oracle function against something independent of its own
formula: library routines, closed forms, brute-force loops, or an
algebraically different evaluation of the same operator."""
import math

import numpy as np

import pytest
import torch
import torch.nn.functional as F

import oracle
from oracle import inputs

torch.manual_seed(0)
F64 = torch.float64


def _rand(*shape, seed=0, dtype=F64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g, dtype=dtype)


# ---------------------------------------------------------------- softmax
@pytest.mark.parametrize("causal", [False, True])
def test_softmax_vs_sdpa(causal):
    q, k, v = _rand(2, 33, 3, 16, seed=1), _rand(2, 33, 3, 16, seed=2), _rand(2, 33, 3, 24, seed=3)
    o, lse = oracle.softmax_attention(q, k, v, causal=causal, compute_dtype=F64, return_lse=True)
    ref = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2),
                                         is_causal=causal).transpose(1, 2)
    torch.testing.assert_close(o, ref, rtol=1e-10, atol=1e-10)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k) / math.sqrt(16)
    if causal:
        s = s.masked_fill(torch.triu(torch.ones(33, 33, dtype=torch.bool), 1), float("-inf"))
    torch.testing.assert_close(lse, torch.logsumexp(s, -1), rtol=1e-10, atol=1e-10)


def test_softmax_closed_forms():
    # constant K: every unmasked score is equal -> causal output = running mean of V
    q, v = _rand(1, 9, 2, 8, seed=4), _rand(1, 9, 2, 5, seed=5)
    k = torch.ones(1, 9, 2, 8, dtype=F64)
    o = oracle.softmax_attention(q, k, v, causal=True, compute_dtype=F64)
    mean = torch.cumsum(v, 1) / torch.arange(1, 10, dtype=F64).view(1, 9, 1, 1)
    torch.testing.assert_close(o, mean, rtol=1e-12, atol=1e-12)
    # S = 1: O = V
    q1, k1, v1 = _rand(2, 1, 2, 8), _rand(2, 1, 2, 8, seed=7), _rand(2, 1, 2, 4, seed=8)
    torch.testing.assert_close(oracle.softmax_attention(q1, k1, v1, compute_dtype=F64), v1)


def test_softmax_bruteforce_tiny():
    q, k, v = _rand(1, 4, 1, 3, seed=9), _rand(1, 4, 1, 3, seed=10), _rand(1, 4, 1, 2, seed=11)
    o = oracle.softmax_attention(q, k, v, causal=True, compute_dtype=F64)
    for i in range(4):
        w = [math.exp(sum(float(q[0, i, 0, d] * k[0, j, 0, d]) for d in range(3)) / math.sqrt(3)) for j in range(i + 1)]
        for d in range(2):
            exp = sum(w[j] * float(v[0, j, 0, d]) for j in range(i + 1)) / sum(w)
            assert abs(float(o[0, i, 0, d]) - exp) < 1e-12


# ---------------------------------------------------------------- sigmoid / relu
def test_sigmoid_closed_form():
    q, k, v = _rand(1, 6, 2, 4, seed=12), _rand(1, 6, 2, 4, seed=13), _rand(1, 6, 2, 3, seed=14)
    for scale, bias in [(1.0, -1.7), (0.5, 0.3)]:
        o = oracle.sigmoid_attention(q, k, v, torch.tensor([bias], dtype=F64), causal=True, softmax_scale=scale, compute_dtype=F64)
        for h in range(2):
            for i in range(6):
                acc = torch.zeros(3, dtype=F64)
                for j in range(i + 1):          # masked entries contribute exactly 0
                    x = float(q[0, i, h] @ k[0, j, h]) * scale + bias
                    acc += v[0, j, h] / (1.0 + math.exp(-x))
                torch.testing.assert_close(o[0, i, h], acc, rtol=1e-12, atol=1e-12)
    # non-causal: every pair contributes
    o = oracle.sigmoid_attention(q, k, v, 0.0, causal=False, compute_dtype=F64)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k)
    torch.testing.assert_close(o, torch.einsum("bhqk,bkhd->bqhd", torch.sigmoid(s), v), rtol=1e-12, atol=1e-12)


def test_relu_bruteforce():
    q, k, v = _rand(1, 5, 2, 4, seed=15), _rand(1, 5, 2, 4, seed=16), _rand(1, 5, 2, 3, seed=17)
    o = oracle.relu_attention(q, k, v, compute_dtype=F64)
    for h in range(2):
        for i in range(5):
            acc = torch.zeros(3, dtype=F64)
            for j in range(5):
                acc += max(float(q[0, i, h] @ k[0, j, h]) / 2.0, 0.0) * v[0, j, h]
            torch.testing.assert_close(o[0, i, h], acc, rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------- retention (parallel, normalised)
def test_retention_decay_mask_values():
    m = oracle.retention_decay_mask(3, 6, F64)[0]
    for h in range(3):
        g = 1 - 2.0 ** (-5 - h)
        for i in range(6):
            for j in range(6):
                exp = g ** (i - j) if i >= j else 0.0
                assert abs(float(m[h, i, j]) - exp) < 1e-14


def test_retention_parallel_bruteforce_and_clamp():
    B, S, H, D, DV = 1, 7, 2, 4, 3
    q, k, v = _rand(B, S, H, D, seed=18), _rand(B, S, H, D, seed=19), _rand(B, S, H, DV, seed=20)
    mask = oracle.retention_decay_mask(H, S, F64)
    for qs in (1.0, 0.01):     # qs=0.01 puts every row sum below 1: clamp active -> un-normalised
        o, r = oracle.retention_parallel(q * qs, k, v, mask, compute_dtype=F64, return_r=True)
        for h in range(H):
            for i in range(S):
                w = [float((q[0, i, h] * qs) @ k[0, j, h]) * float(mask[0, h, i, j]) for j in range(S)]
                rr = max(sum(abs(x) for x in w), 1.0)
                exp = sum((w[j] / rr) * v[0, j, h] for j in range(S))
                torch.testing.assert_close(o[0, i, h], exp, rtol=1e-12, atol=1e-12)
                assert abs(float(r[0, h, i]) - rr) < 1e-12
        if qs == 0.01:
            assert float(r.max()) == 1.0
    # all-ones causal mask: plain causal linear attention / max(sum|qk|,1)
    ones = torch.tril(torch.ones(S, S, dtype=F64)).expand(1, H, S, S)
    o = oracle.retention_parallel(q, k, v, ones, compute_dtype=F64)
    s = torch.einsum("bqhd,bkhd->bhqk", q, k).tril()
    ref = torch.einsum("bhqk,bkhd->bqhd", s / s.abs().sum(-1, keepdim=True).clamp(min=1), v)
    torch.testing.assert_close(o, ref, rtol=1e-12, atol=1e-12)


def test_retention_gradient_with_the_row_scale_held_constant():
    """The gradient the reference's retention operator defines (OnlineRetention.backward,
    examples/retention_parallel.py:76-86: p = scores / r, dscores = dp / r, and the score_mod's factor M):
    dq = ((dO V^T) * M / r) K, dk = ((dO V^T) * M / r)^T Q, dv = P^T dO, written out with einsum, against autograd over
    the oracle with freeze_r; and where the clamp holds r at 1 that is the true gradient."""
    B, S, H, D, DV = 2, 9, 2, 4, 3
    q, k, v, do = _rand(B, S, H, D, seed=30), _rand(B, S, H, D, seed=31), _rand(B, S, H, DV, seed=32), _rand(B, S, H, DV, seed=33)
    mask = oracle.retention_decay_mask(H, S, F64)
    for qs in (3.0, 0.01):
        qq = q * qs
        got = oracle.attention_grads(oracle.retention_parallel, qq, k, v, do, mask=mask, freeze_r=True)
        s_ = torch.einsum("bqhd,bkhd->bhqk", qq, k) * mask
        r = s_.abs().sum(-1, keepdim=True).clamp(min=1)
        assert bool((r > 1).any()) == (qs == 3.0)
        dp = torch.einsum("bqhe,bkhe->bhqk", do, v)
        ds = dp * mask / r
        exp = (torch.einsum("bhqk,bkhd->bqhd", ds, k), torch.einsum("bhqk,bqhd->bkhd", ds, qq), torch.einsum("bhqk,bqhe->bkhe", s_ / r, do))
        for a, b in zip(got, exp):
            torch.testing.assert_close(a, b, rtol=1e-11, atol=1e-11)
        true = oracle.attention_grads(oracle.retention_parallel, qq, k, v, do, mask=mask)
        if qs == 0.01:
            for a, b in zip(got, true):
                torch.testing.assert_close(a, b, rtol=1e-11, atol=1e-11)
        else:
            assert not torch.allclose(got[0], true[0], rtol=1e-3, atol=1e-3)    # r does depend on q and k there


# ---------------------------------------------------------------- RetNet chunked
def test_retnet_three_way():
    B, H, T, Dk, Dv = 1, 3, 64, 8, 6
    q, k, v = _rand(B, H, T, Dk, seed=21), _rand(B, H, T, Dk, seed=22), _rand(B, H, T, Dv, seed=23)
    quad = oracle.retnet_quadratic(q, k, v, compute_dtype=F64)
    rec = oracle.retnet_recurrence(q, k, v, compute_dtype=F64)
    torch.testing.assert_close(quad, rec, rtol=1e-10, atol=1e-10)
    gam = (1 - torch.exp2(-5.0 - torch.arange(H, dtype=F64))).view(1, H, 1).expand(B, H, T)
    for chunk in (8, 16, 64):
        ch = oracle.linear_attention_chunked(q, k, v, torch.log(gam), chunk=chunk, q_scale=Dk ** -0.5, compute_dtype=F64)
        torch.testing.assert_close(ch, rec, rtol=1e-10, atol=1e-10)


# ---------------------------------------------------------------- Mamba2
def test_ssd_three_way():
    b, l, h, p, n = 2, 64, 4, 5, 6
    x = _rand(b, l, h, p, seed=24)
    Bm, Cm = _rand(b, l, 1, n, seed=25), _rand(b, l, 1, n, seed=26)
    dt = F.softplus(_rand(b, l, h, seed=27) - 2)
    A = -torch.exp(torch.rand(h, dtype=F64) * math.log(16))
    seq = oracle.ssd_sequential(x, dt, A, Bm, Cm)
    for chunk in (8, 16, 64):
        ch = oracle.ssd_chunk_scan_combined(x, dt, A, Bm, Cm, chunk_size=chunk, compute_dtype=F64)
        torch.testing.assert_close(ch, seq, rtol=1e-9, atol=1e-9)
    # the operator's view of the same computation (q=C, k=B, v=x*dt, log decay = dt*A), BHSD
    lin = oracle.linear_attention_chunked(
        Cm.permute(0, 2, 1, 3), Bm.permute(0, 2, 1, 3), x.permute(0, 2, 1, 3),
        (dt * A).permute(0, 2, 1), chunk=16, v_scale=dt.permute(0, 2, 1), compute_dtype=F64)
    torch.testing.assert_close(lin.permute(0, 2, 1, 3), seq, rtol=1e-9, atol=1e-9)


def test_ssd_two_groups():
    b, l, h, p, n = 1, 32, 4, 3, 4
    x, Bm, Cm = _rand(b, l, h, p, seed=28), _rand(b, l, 2, n, seed=29), _rand(b, l, 2, n, seed=30)
    dt = F.softplus(_rand(b, l, h, seed=31))
    A = -torch.rand(h, dtype=F64) - 0.5
    torch.testing.assert_close(oracle.ssd_chunk_scan_combined(x, dt, A, Bm, Cm, 8, F64),
                               oracle.ssd_sequential(x, dt, A, Bm, Cm), rtol=1e-9, atol=1e-9)


# ---------------------------------------------------------------- gated retention
def test_simple_gla_vs_recurrence():
    B, H, T, Dk, Dv = 1, 2, 48, 8, 5
    q, k, v = _rand(B, H, T, Dk, seed=32), _rand(B, H, T, Dk, seed=33), _rand(B, H, T, Dv, seed=34)
    g = F.logsigmoid(_rand(B, H, T, seed=35)).clamp_min(-5)
    rec = oracle.simple_gla_recurrence(q, k, v, g)
    for chunk in (8, 16, 48):
        torch.testing.assert_close(oracle.simple_gla_chunked(q, k, v, g, chunk, compute_dtype=F64), rec,
                                   rtol=1e-10, atol=1e-10)


# ---------------------------------------------------------------- MLA decode
def test_mla_vs_sdpa_and_split_invariance():
    B, Hq, Skv, d, dpe = 2, 6, 40, 16, 4
    q, q_pe = _rand(B, 1, Hq, d, seed=36), _rand(B, 1, Hq, dpe, seed=37)
    kv, k_pe = _rand(B, Skv, 1, d, seed=38), _rand(B, Skv, 1, dpe, seed=39)
    o, lse = oracle.mla_decode(q, q_pe, kv, k_pe, compute_dtype=F64, return_lse=True)
    qq = torch.cat([q, q_pe], -1).transpose(1, 2)                      # [B,Hq,1,d+dpe]
    kk = torch.cat([kv, k_pe], -1).transpose(1, 2).expand(B, Hq, Skv, d + dpe)
    vv = kv.transpose(1, 2).expand(B, Hq, Skv, d)
    # sdpa's default scale 1/sqrt(E) with E = d + dpe is the scale the operator uses
    ref = F.scaled_dot_product_attention(qq, kk, vv).transpose(1, 2)
    torch.testing.assert_close(o, ref, rtol=1e-10, atol=1e-10)
    # split-KV + log-sum-exp merge reproduces the whole
    parts = [oracle.mla_decode(q, q_pe, kv[:, s], k_pe[:, s], compute_dtype=F64, return_lse=True)
             for s in (slice(0, 8), slice(8, 24), slice(24, 40))]
    lses = torch.stack([p[1] for p in parts])                         # [3,B,Hq]
    tot = torch.logsumexp(lses, 0)
    merged = sum(p[0] * torch.exp(p[1] - tot).view(B, 1, Hq, 1) for p in parts)
    torch.testing.assert_close(merged, o, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(tot, lse, rtol=1e-10, atol=1e-10)


# ---------------------------------------------------------------- helpers
def test_assert_close_rule():
    a = torch.zeros(1000)
    e = torch.zeros(1000)
    e[:5] = 1.0
    with pytest.raises(AssertionError):
        oracle.assert_close(a, e, rtol=1e-2, atol=1e-2)
    oracle.assert_close(a, e, rtol=1e-2, atol=1e-2, mismatch_ratio=5e-3)
    with pytest.raises(AssertionError):
        oracle.assert_close(a, e, rtol=1e-2, atol=1e-2, mismatch_ratio=4e-3)


def test_input_generators_are_seeded():
    a = inputs.softmax_inputs(1, 2, 8, 4, 4, seed=3)
    b = inputs.softmax_inputs(1, 2, 8, 4, 4, seed=3)
    for x, y in zip(a, b):
        assert torch.equal(x, y) and x.dtype == torch.bfloat16
    Cm, Bm, x, dt, A = inputs.mamba2_inputs(1, 4, 16, 8, 8)
    assert Cm.shape == (1, 1, 16, 8) and x.shape == (1, 4, 16, 8) and dt.dtype == torch.float32
    assert (A < 0).all() and (A >= -16).all() and (dt > 0).all()


def test_grouped_query_equals_repeated_kv_heads():
    """Hkv < H: query head h reads kv head h // (H // Hkv), i.e. the multi-head result on k, v with every
    kv head repeated H // Hkv times."""
    g = torch.Generator().manual_seed(4)
    B, S, H, Hkv, D = 2, 40, 6, 2, 16
    q = torch.randn(B, S, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, S, Hkv, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, S, Hkv, D, generator=g, dtype=torch.float64)
    kr, vr = k.repeat_interleave(H // Hkv, dim=2), v.repeat_interleave(H // Hkv, dim=2)
    kw = dict(compute_dtype=torch.float64)
    torch.testing.assert_close(oracle.softmax_attention(q, k, v, causal=True, **kw), oracle.softmax_attention(q, kr, vr, causal=True, **kw))
    torch.testing.assert_close(oracle.sigmoid_attention(q, k, v, 0.3, causal=True, **kw), oracle.sigmoid_attention(q, kr, vr, 0.3, causal=True, **kw))
    torch.testing.assert_close(oracle.relu_attention(q, k, v, **kw), oracle.relu_attention(q, kr, vr, **kw))
    sd = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2), kr.transpose(1, 2), vr.transpose(1, 2), is_causal=True)
    torch.testing.assert_close(oracle.softmax_attention(q, k, v, causal=True, **kw), sd.transpose(1, 2))


def test_attention_grads_vs_finite_differences_and_sdpa():
    """The gradient oracle is autograd over the pinned fp64 forward; checked against central
    differences along random directions and, for softmax, against SDPA's own backward."""
    g = torch.Generator().manual_seed(9)
    B, S, H, Hkv, D, DV = 1, 12, 4, 2, 8, 6
    q = torch.randn(B, S, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, S, Hkv, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, S, Hkv, DV, generator=g, dtype=torch.float64)
    dout = torch.randn(B, S, H, DV, generator=g, dtype=torch.float64)
    cases = [(oracle.softmax_attention, dict(causal=True)), (oracle.sigmoid_attention, dict(bias=-0.7, causal=True, softmax_scale=0.3)),
             (oracle.relu_attention, dict()),
             # (the additive-term form the backward kernels of the softmax family are checked against)
             (oracle.biased_attention, dict(add=torch.randn(B, H, S, S, generator=g, dtype=torch.float64), causal=True, softmax_scale=0.3)),
             (oracle.biased_attention, dict(add=torch.randn(1, H, 1, S, generator=g, dtype=torch.float64), causal=True,
                                            softmax_scale=0.4, bias=0.2, softcap=1.5))]
    for fwd, kw in cases:
        dq, dk, dv = oracle.attention_grads(fwd, q, k, v, dout, **kw)
        f = lambda q_, k_, v_: float((fwd(q_, k_, v_, compute_dtype=torch.float64, **kw) * dout).sum())
        for t, grad, idx in ((q, dq, 0), (k, dk, 1), (v, dv, 2)):
            direction = torch.randn(t.shape, generator=g, dtype=torch.float64)
            eps = 1e-6
            args_p, args_m = [q, k, v], [q, k, v]
            args_p[idx], args_m[idx] = t + eps * direction, t - eps * direction
            fd = (f(*args_p) - f(*args_m)) / (2 * eps)
            assert abs(fd - float((grad * direction).sum())) < 1e-5 * max(1.0, abs(fd)), (fwd.__name__, idx)
    qs, ks, vs = (t.clone().requires_grad_(True) for t in (q, k, v))
    o = torch.nn.functional.scaled_dot_product_attention(qs.transpose(1, 2), ks.repeat_interleave(2, dim=2).transpose(1, 2),
                                                         vs.repeat_interleave(2, dim=2).transpose(1, 2), is_causal=True)
    o.transpose(1, 2).backward(dout)
    dq, dk, dv = oracle.attention_grads(oracle.softmax_attention, q, k, v, dout, causal=True)
    for a, b in ((dq, qs.grad), (dk, ks.grad), (dv, vs.grad)):
        torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-9)
    # an additive tile is SDPA's float attn_mask
    add = torch.randn(B, H, S, S, generator=g, dtype=torch.float64)
    qs, ks, vs = (t.clone().requires_grad_(True) for t in (q, k, v))
    o = torch.nn.functional.scaled_dot_product_attention(qs.transpose(1, 2), ks.repeat_interleave(2, dim=2).transpose(1, 2),
                                                         vs.repeat_interleave(2, dim=2).transpose(1, 2), attn_mask=add)
    o.transpose(1, 2).backward(dout)
    dq, dk, dv = oracle.attention_grads(oracle.biased_attention, q, k, v, dout, add=add)
    for a, b in ((dq, qs.grad), (dk, ks.grad), (dv, vs.grad)):
        torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-9)


def test_linear_attention_grads_vs_finite_differences():
    g = torch.Generator().manual_seed(11)
    B, Hq, H, T, Dk, Dv = 1, 1, 2, 24, 6, 5
    q = torch.randn(B, Hq, T, Dk, generator=g, dtype=torch.float64)
    k = torch.randn(B, Hq, T, Dk, generator=g, dtype=torch.float64)
    v = torch.randn(B, H, T, Dv, generator=g, dtype=torch.float64)
    ld = -torch.rand(B, H, T, generator=g, dtype=torch.float64)
    vs = torch.rand(B, H, T, generator=g, dtype=torch.float64) + 0.5
    dout = torch.randn(B, H, T, Dv, generator=g, dtype=torch.float64)
    grads = oracle.linear_attention_grads(q, k, v, ld, dout, q_scale=0.4, v_scale=vs, chunk=8)
    args = [q, k, v, ld, vs]
    f = lambda a: float((oracle.linear_attention_chunked(a[0], a[1], a[2], a[3], chunk=8, q_scale=0.4, v_scale=a[4],
                                                         compute_dtype=torch.float64) * dout).sum())
    for idx, grad in enumerate(grads):
        direction = torch.randn(args[idx].shape, generator=g, dtype=torch.float64)
        eps = 1e-6
        ap, am = list(args), list(args)
        ap[idx], am[idx] = args[idx] + eps * direction, args[idx] - eps * direction
        fd = (f(ap) - f(am)) / (2 * eps)
        assert abs(fd - float((grad * direction).sum())) < 1e-5 * max(1.0, abs(fd)), idx


def test_sparse_decode_equals_dense_attention_over_kept_keys():
    g = torch.Generator().manual_seed(13)
    B, H, G, S, D, bs = 2, 4, 2, 96, 16, 32
    q = torch.randn(B, 1, H, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, S, G, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, S, G, D, generator=g, dtype=torch.float64)
    bm = torch.tensor([[[1, 0, 1], [0, 1, 1]], [[1, 1, 0], [1, 0, 0]]], dtype=torch.bool)
    lens = torch.tensor([96, 70], dtype=torch.int32)
    got = oracle.sparse_decode_attention(q, k, v, bm, lens, block_size=bs, compute_dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            gi = h // (H // G)
            idx = [n for n in range(S) if bm[b, gi, n // bs] and n < int(lens[b])]
            ref = oracle.softmax_attention(q[b:b + 1, :, h:h + 1], k[b:b + 1, idx, gi:gi + 1], v[b:b + 1, idx, gi:gi + 1], causal=False,
                                           compute_dtype=torch.float64)
            torch.testing.assert_close(got[b, h], ref[0, 0, 0])


def test_paged_mla_identity_table_and_page_permutation():
    g = torch.Generator().manual_seed(17)
    B, Hq, page, npg = 2, 3, 4, 5
    q = torch.randn(B, 1, Hq, 24, generator=g, dtype=torch.float64)
    cache = torch.randn(B * npg, page, 1, 24, generator=g, dtype=torch.float64)
    table = torch.arange(B * npg, dtype=torch.int32).view(B, npg)
    lens = torch.tensor([20, 13], dtype=torch.int32)
    out, lse = oracle.paged_mla_decode(q, cache, table, lens, head_dim_v=16, compute_dtype=torch.float64)
    for b in range(B):
        rows = cache[b * npg:(b + 1) * npg].reshape(1, -1, 1, 24)[:, :int(lens[b])]
        o, l = oracle.mla_decode(q[b:b + 1, :, :, :16], q[b:b + 1, :, :, 16:], rows[..., :16], rows[..., 16:], compute_dtype=torch.float64,
                                 return_lse=True)
        torch.testing.assert_close(out[b:b + 1], o)
        torch.testing.assert_close(lse[b, :, 0], l[0])
    perm = torch.randperm(B * npg, generator=g)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(B * npg)
    out2, lse2 = oracle.paged_mla_decode(q, cache[perm], inv[table.long()].to(torch.int32), lens, head_dim_v=16, compute_dtype=torch.float64)
    torch.testing.assert_close(out2, out)
    torch.testing.assert_close(lse2, lse)


def test_masked_attention_against_sdpa_and_special_cases():
    g = torch.Generator().manual_seed(19)
    B, H, S, D = 2, 3, 24, 8
    q, k, v = (torch.randn(B, S, H, D, generator=g, dtype=torch.float64) for _ in range(3))
    keep = torch.rand(B, H, S, S, generator=g) < 0.4
    keep[0, 1, 5] = False                                   # a row without any key
    got = oracle.masked_attention(q, k, v, keep=keep, compute_dtype=torch.float64)
    sd = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), attn_mask=keep)
    sd = torch.nan_to_num(sd, nan=0.0).transpose(1, 2)      # SDPA gives NaN for the empty row
    assert keep.any(-1).all(-1).tolist() != [[True] * H] * B
    torch.testing.assert_close(got, sd)
    assert torch.equal(got[0, 5, 1], torch.zeros(D, dtype=torch.float64))
    # the lower-triangular keep mask is the causal operator; a broadcast mask is the same for every (batch, head)
    tril = torch.tril(torch.ones(S, S, dtype=torch.bool)).view(1, 1, S, S)
    torch.testing.assert_close(oracle.masked_attention(q, k, v, keep=tril, compute_dtype=torch.float64),
                               oracle.softmax_attention(q, k, v, causal=True, compute_dtype=torch.float64))
    # a block mask: every query block attends to the gathered keys of its kept blocks only
    bm = torch.tensor([[1, 0, 1], [0, 0, 0], [0, 1, 1], [1, 1, 1]], dtype=torch.int8).view(1, 1, 4, 3).expand(B, H, 4, 3)
    got = oracle.masked_attention(q, k, v, block_mask=bm, compute_dtype=torch.float64)
    for qb in range(4):
        rows = slice(qb * 6, qb * 6 + 6)
        idx = [n for n in range(S) if bm[0, 0, qb, n // 8]]
        if not idx:
            assert torch.count_nonzero(got[:, rows]) == 0
            continue
        ref = oracle.softmax_attention(q[:, rows], k[:, idx], v[:, idx], causal=False, compute_dtype=torch.float64)
        torch.testing.assert_close(got[:, rows], ref)
    # sigmoid / relu: element by element
    for family, fn in (("sigmoid", lambda x: 1 / (1 + math.exp(-(x - 0.3)))), ("relu", lambda x: max(x, 0.0))):
        got = oracle.masked_attention(q[:1, :6, :1], k[:1, :6, :1], v[:1, :6, :1], keep=keep[:1, :1, :6, :6], family=family,
                                      softmax_scale=0.5, bias=-0.3, compute_dtype=torch.float64)
        for i in range(6):
            acc = torch.zeros(D, dtype=torch.float64)
            for j in range(6):
                if keep[0, 0, i, j]:
                    acc += fn(0.5 * float(q[0, i, 0] @ k[0, j, 0])) * v[0, j, 0]
            torch.testing.assert_close(got[0, i, 0], acc)


def test_mla_work_plan_small_cases_and_invariants():
    # two entries of 3 and 1 blocks on two parts: total = (3+5) + (1+5) = 14, payload = max(7 + 5, 10) = 12;
    # part 0 takes entry 0 whole (8) and has 4 left, not enough for entry 1 (6) nor for one block beside the overhead
    meta, splits = oracle.mla_work_plan([192, 64], parts=2)
    assert meta[:, :5].tolist() == [[0, 0, 0, 192, 0], [1, 0, 1, 64, 0]] and splits.tolist() == [0, 1, 2]
    # one entry of 40 blocks on 4 parts: payload = max(ceil(45/4) + 5, 10) = 17 -> pieces of 12 blocks, the last of 4
    meta, splits = oracle.mla_work_plan([40 * 64], parts=4)
    assert meta[:, :5].tolist() == [[0, 0, 0, 768, 0], [0, 768, 0, 1536, 1], [0, 1536, 0, 2304, 2], [0, 2304, 0, 2560, 3]]
    assert splits.tolist() == [0, 4]
    # more parts than work: the surplus parts start at batch == B and are empty
    meta, splits = oracle.mla_work_plan([64], parts=3)
    assert meta[0, :5].tolist() == [0, 0, 0, 64, 0] and meta[1, 0] == 1 and meta[2, 0] == 1 and splits.tolist() == [0, 1]
    rng = np.random.default_rng(0)
    for _ in range(200):
        B = int(rng.integers(1, 40))
        lens = rng.integers(0, 5000, size=B)
        parts = int(rng.integers(1, 300))
        meta, splits = oracle.mla_work_plan(lens, parts)
        pieces = oracle.plan_pieces(meta, splits, lens)
        payload = max(-(-sum(-(-int(x) // 64) + 5 for x in lens) // parts) + 5, 10)
        cover = {b: [] for b in range(B)}
        load = {}
        for p, b, begin, end, sidx in pieces:
            assert sidx == len(cover[b])                                    # split indices count up per batch entry
            cover[b].append((begin, end))
            load[p] = load.get(p, 0) + -(-(end - begin) // 64) + 5
        for b in range(B):
            assert cover[b][0][0] == 0 and cover[b][-1][1] == lens[b]       # every token exactly once, in order
            assert all(a[1] == c[0] for a, c in zip(cover[b], cover[b][1:]))
            assert all(e > s_ for s_, e in cover[b]) or lens[b] == 0
            assert splits[b + 1] - splits[b] == len(cover[b])
        assert all(v <= payload for v in load.values())


def test_biased_attention_against_sdpa_and_special_cases():
    g = torch.Generator().manual_seed(23)
    B, H, S, D = 2, 3, 20, 8
    q, k, v = (torch.randn(B, S, H, D, generator=g, dtype=torch.float64) for _ in range(3))
    add = torch.randn(B, H, S, S, generator=g, dtype=torch.float64)
    qt, kt, vt = (t.transpose(1, 2) for t in (q, k, v))
    # a float attn_mask is added to the scaled scores by SDPA
    got, lse = oracle.biased_attention(q, k, v, add=add, compute_dtype=torch.float64, return_lse=True)
    sd = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=add).transpose(1, 2)
    torch.testing.assert_close(got, sd)
    x = torch.einsum("bqhd,bkhd->bhqk", q, k) / math.sqrt(D) + add
    torch.testing.assert_close(lse, torch.logsumexp(x, dim=-1))
    # with the causal triangle: the same as a float mask that also holds -inf above the diagonal
    tri = torch.full((S, S), float("-inf"), dtype=torch.float64).triu(1)
    got = oracle.biased_attention(q, k, v, add=add, causal=True, compute_dtype=torch.float64)
    sd = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=add + tri).transpose(1, 2)
    torch.testing.assert_close(got, sd)
    # broadcast shapes: a [heads, 1, 1]-shaped slope times (kv - q) (ALiBi), a per-row tensor, a kv vector
    idx = torch.arange(S, dtype=torch.float64)
    alibi = torch.tensor([0.5, 0.25, 0.125], dtype=torch.float64).view(1, H, 1, 1) * (idx.view(1, 1, 1, S) - idx.view(1, 1, S, 1))
    got = oracle.biased_attention(q, k, v, add=alibi, causal=True, compute_dtype=torch.float64)
    sd = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=alibi.expand(B, H, S, S) + tri).transpose(1, 2)
    torch.testing.assert_close(got, sd)
    row = torch.randn(B, H, S, 1, generator=g, dtype=torch.float64)      # constant along the row: softmax ignores it, lse moves by it
    base, lse0 = oracle.softmax_attention(q, k, v, causal=True, compute_dtype=torch.float64, return_lse=True)
    got, lse = oracle.biased_attention(q, k, v, add=row, causal=True, compute_dtype=torch.float64, return_lse=True)
    torch.testing.assert_close(got, base)
    torch.testing.assert_close(lse, lse0 + row.squeeze(-1))
    torch.testing.assert_close(oracle.biased_attention(q, k, v, causal=False, compute_dtype=torch.float64),
                               oracle.softmax_attention(q, k, v, causal=False, compute_dtype=torch.float64))
    # soft-capping, sigmoid, relu: element by element
    colv = torch.randn(S, generator=g, dtype=torch.float64)
    for family, cap in (("softmax", 2.5), ("sigmoid", None), ("relu", None)):
        got = oracle.biased_attention(q[:1, :5, :1], k[:1, :5, :1], v[:1, :5, :1], add=colv[:5].view(1, 1, 1, 5), causal=True, family=family,
                                      softmax_scale=0.7, bias=-0.2, softcap=cap, compute_dtype=torch.float64)
        for i in range(5):
            w = []
            for j in range(i + 1):
                x = float(q[0, i, 0] @ k[0, j, 0]) * 0.7 - 0.2 + float(colv[j])
                if cap is not None:
                    x = cap * math.tanh(x)
                w.append(math.exp(x) if family == "softmax" else (1 / (1 + math.exp(-x)) if family == "sigmoid" else max(x, 0.0)))
            tot = sum(w) if family == "softmax" else 1.0
            ref = sum(wj / tot * v[0, j, 0] for j, wj in enumerate(w))
            torch.testing.assert_close(got[0, i, 0], ref)
