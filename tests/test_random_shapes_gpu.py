"""Seeded random sweep over shapes, strides, head groupings and lengths for every C-ABI entry point,
each case against the CPU oracle (atol 2e-2 / rtol 1e-2; un-normalised families with the allowance
their dedicated tests state).  Sizes stay small so the oracle finishes in seconds."""
import math
import random

import pytest
import torch

import oracle
from oracle import inputs

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


def _hb():
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    return hb


def _packed(B, S, H, D, g, dtype, gain=1.0):
    """A [B,S,H,D] view with non-trivial strides: a slice of a wider buffer (as q, k, v cut out of one packed projection)."""
    pad_h, pad_d = random.choice([0, 1, 2]), random.choice([0, 8, 64])
    buf = (gain * torch.randn(B, S, H + pad_h, D + pad_d, generator=g)).to(dtype)
    return buf[:, :, pad_h // 2: pad_h // 2 + H, :D] if pad_d or pad_h else buf


@pytest.mark.parametrize("seed", range(24))
def test_parallel_forward_random(seed):
    hb = _hb()
    random.seed(seed)
    g = torch.Generator().manual_seed(seed)
    D, DV = random.choice([(128, 128), (128, 128), (64, 64), (128, 256), (256, 256), (192, 128)])
    family = random.choice(["softmax", "softmax", "sigmoid", "relu"])
    dtype = random.choice([torch.bfloat16, torch.float16])
    B, Hkv, grp = random.randint(1, 3), random.randint(1, 3), random.choice([1, 1, 2, 4])
    H = Hkv * grp
    causal = random.random() < 0.6
    Sq = random.choice([1, 17, 64, 100, 128, 257, 300, 511])
    Skv = Sq if causal else random.choice([Sq, 1, 33, 200, 640])
    q = _packed(B, Sq, H, D, g, dtype)
    k = _packed(B, Skv, Hkv, D, g, dtype, 0.5)
    v = _packed(B, Skv, Hkv, DV, g, dtype, 0.5)
    scale = 1 / math.sqrt(D)
    print(f"seed {seed}: {family} D{D}/{DV} B{B} H{H}/{Hkv} Sq{Sq} Skv{Skv} causal={causal} {dtype} strides q{q.stride()} k{k.stride()}", flush=True)
    qc, kc, vc = q.cuda(), k.cuda(), v.cuda()
    # .cuda() of a strided view is contiguous: rebuild the same strides on the device
    def dev(t):
        d = torch.empty_strided(t.shape, t.stride(), dtype=t.dtype, device="cuda")
        d.copy_(t)
        return d
    qc, kc, vc = dev(q), dev(k), dev(v)
    if family == "softmax":
        lse = torch.full((B, H, Sq), float("nan"), device="cuda")
        o = hb.attn_fwd(qc, kc, vc, family=hb.MA_ATTN_SOFTMAX, causal=causal, scale=scale, row_scale=lse)
        ref, lse_ref = oracle.softmax_attention(q, k, v, causal=causal, return_lse=True)
        torch.cuda.synchronize()
        torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-3, atol=1e-3)
        oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    elif family == "sigmoid":
        bias = -math.log(max(Skv, 2))
        o = hb.attn_fwd(qc, kc, vc, family=hb.MA_ATTN_SIGMOID, causal=causal, scale=scale, bias=bias)
        torch.cuda.synchronize()
        oracle.assert_close(o.float().cpu(), oracle.sigmoid_attention(q, k, v, bias, causal=causal, softmax_scale=scale), rtol=RTOL, atol=ATOL)
    else:
        o = hb.attn_fwd(qc, kc, vc, family=hb.MA_ATTN_RELU, causal=causal, scale=scale)
        torch.cuda.synchronize()
        ref = oracle.relu_attention(q, k, v) if not causal else None
        if ref is None:      # causal relu: zero fill, defined through the masked sigmoid-style sum
            keep = torch.arange(Sq).view(-1, 1) >= torch.arange(Skv).view(1, -1)
            ref = torch.empty(B, Sq, H, DV)
            for b in range(B):
                for h in range(H):
                    s = torch.relu(q[b, :, h].float() @ k[b, :, h // grp].float().T * scale) * keep
                    ref[b, :, h] = s @ v[b, :, h // grp].float()
        oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3)
        oracle.assert_close(o.float().cpu(), ref, rtol=1e-1, atol=1e-1, mismatch_ratio=1e-3)


@pytest.mark.parametrize("seed", range(12))
def test_parallel_backward_random(seed):
    hb = _hb()
    random.seed(100 + seed)
    g = torch.Generator().manual_seed(100 + seed)
    D, DV = random.choice([(128, 128), (64, 64), (128, 256), (192, 128)])
    family = random.choice(["softmax", "softmax", "sigmoid", "relu"])
    dtype = random.choice([torch.bfloat16, torch.float16])
    B, Hkv, grp = random.randint(1, 2), random.randint(1, 2), random.choice([1, 2, 3])
    H = Hkv * grp
    causal = family != "relu" and random.random() < 0.6
    Sq = random.choice([1, 31, 64, 100, 129, 300])
    Skv = Sq if causal else random.choice([Sq, 33, 200])
    q = torch.randn(B, Sq, H, D, generator=g).to(dtype)
    k = (0.5 * torch.randn(B, Skv, Hkv, D, generator=g)).to(dtype)
    v = (0.5 * torch.randn(B, Skv, Hkv, DV, generator=g)).to(dtype)
    dout = (0.5 * torch.randn(B, Sq, H, DV, generator=g)).to(dtype)
    scale, bias = 1 / math.sqrt(D), (-1.5 if family == "sigmoid" else 0.0)
    fam = {"softmax": hb.MA_ATTN_SOFTMAX, "sigmoid": hb.MA_ATTN_SIGMOID, "relu": hb.MA_ATTN_RELU}[family]
    print(f"seed {seed}: bwd {family} D{D}/{DV} B{B} H{H}/{Hkv} Sq{Sq} Skv{Skv} causal={causal} {dtype}", flush=True)
    lse = torch.empty(B, H, Sq, device="cuda") if family == "softmax" else None
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=fam, causal=causal, scale=scale, bias=bias, row_scale=lse)
    got = hb.attn_bwd(q.cuda(), k.cuda(), v.cuda(), o, dout.cuda(), lse, family=fam, causal=causal, scale=scale, bias=bias)
    torch.cuda.synchronize()
    if family == "softmax":
        ref = oracle.attention_grads(oracle.softmax_attention, q, k, v, dout, causal=causal, softmax_scale=scale)
    elif family == "sigmoid":
        ref = oracle.attention_grads(oracle.sigmoid_attention, q, k, v, dout, bias=bias, causal=causal, softmax_scale=scale)
    else:
        ref = oracle.attention_grads(oracle.relu_attention, q, k, v, dout, softmax_scale=scale)
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        oracle.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3, msg=name)


@pytest.mark.parametrize("seed", range(16))
def test_linear_forward_random(seed):
    hb = _hb()
    random.seed(200 + seed)
    g = torch.Generator().manual_seed(200 + seed)
    Dk = random.choice([128, 256])
    Dv = random.choice([64, 128, 192, 256, 512])
    B, Hq, rep = random.randint(1, 2), random.randint(1, 2), random.choice([1, 1, 2, 4])
    H = Hq * rep
    T = random.choice([1, 31, 32, 100, 256, 300, 515])
    segments = random.choice([0, 1, 2, 5])
    use_vs = random.random() < 0.5
    q = torch.randn(B, Hq, T, Dk, generator=g).bfloat16()
    k = (0.1 * torch.randn(B, Hq, T, Dk, generator=g)).bfloat16()
    v = torch.randn(B, H, T, Dv, generator=g).bfloat16()
    ld = torch.nn.functional.logsigmoid(torch.randn(B, H, T, generator=g) + 3.0)
    vs = torch.rand(B, H, T, generator=g) + 0.5 if use_vs else None
    print(f"seed {seed}: linear Dk{Dk} Dv{Dv} B{B} H{H}/{Hq} T{T} segments={segments} v_scale={use_vs}", flush=True)
    o = hb.linear_fwd(q.cuda(), k.cuda(), v.cuda(), ld.cuda(), q_scale=Dk ** -0.5, v_scale=vs.cuda() if use_vs else None, segments=segments)
    torch.cuda.synchronize()
    chunk = T if T < 64 or T % 32 else 32
    ref = oracle.linear_attention_chunked(q, k, v, ld, chunk=chunk, q_scale=Dk ** -0.5, v_scale=vs)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("seed", range(10))
def test_mla_random(seed):
    hb = _hb()
    random.seed(300 + seed)
    B, Hq = random.randint(1, 4), random.choice([1, 7, 16, 40, 128, 130])
    Skv = random.choice([1, 31, 64, 100, 500, 1023, 2048])
    ns = min(random.choice([0, 1, 2, 3, 5]), (Skv + 63) // 64)      # the library refuses more splits than 64-row tiles
    dtype = random.choice([torch.bfloat16, torch.float16])
    q, q_pe, kv, k_pe = inputs.mla_inputs(B, Hq, Skv, 512, 64, dtype=dtype, seed=300 + seed)
    # the fused-cache layout: kv and k_pe as strided views of one [B,Skv,1,576] buffer
    cache = torch.cat([kv, k_pe], dim=-1).cuda()
    print(f"seed {seed}: mla B{B} Hq{Hq} Skv{Skv} ns{ns} {dtype}", flush=True)
    lse = torch.full((B, Hq), float("nan"), device="cuda")
    o = hb.mla_decode(q.cuda(), q_pe.cuda(), cache[..., :512], cache[..., 512:], scale=1 / math.sqrt(576), num_split=ns, lse=lse)
    torch.cuda.synchronize()
    ref, lse_ref = oracle.mla_decode(q, q_pe, kv, k_pe, return_lse=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-4, atol=1e-4)
