"""Seeded synthetic inputs for the five benchmark configurations (test
infrastructure only).  Values are drawn on the CPU from a fixed
``torch.Generator`` so the CPU oracle and the GPU operator see identical
numbers; bf16 tensors are rounded once here and the oracle consumes the rounded
values."""
from __future__ import annotations

import math

import torch

CONFIGS = {
    # name: full-size shape parameters quoted by the benchmark definition
    "c1_softmax_fp32": dict(B=1, H=4, S=512, D=64, DV=64, causal=False, dtype=torch.float32),
    "c2_softmax_causal": dict(B=8, H=32, S=4096, D=128, DV=128, causal=True, dtype=torch.bfloat16),
    "c3_retnet": dict(B=8, H=16, S=2048, D=256, DV=512, chunk=64, dtype=torch.bfloat16),
    "c4_mamba2": dict(B=8, H=64, S=2048, P=64, N=128, chunk=256, dtype=torch.bfloat16),
    "c5_mla_decode": dict(B=64, HQ=128, SKV=4096, D=512, DPE=64, dtype=torch.bfloat16),
}


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def softmax_inputs(B, H, S, D, DV, dtype=torch.bfloat16, seed=0):
    """q,k,v ~ N(0,1) in BSHD."""
    g = _gen(seed)
    q = torch.randn(B, S, H, D, generator=g).to(dtype)
    k = torch.randn(B, S, H, D, generator=g).to(dtype)
    v = torch.randn(B, S, H, DV, generator=g).to(dtype)
    return q, k, v


def retnet_inputs(B, H, S, D, DV, dtype=torch.bfloat16, seed=0, layout="bhsd"):
    """q,k ~ N(0,1)/sqrt(D), v ~ N(0,1); decay gamma_h = 1-2^(-5-h) broadcast
    to [B,H,S] fp32 (the operator's ``decay`` argument)."""
    g = _gen(seed)
    shp = (B, H, S) if layout == "bhsd" else (B, S, H)
    q = (torch.randn(*shp, D, generator=g) / math.sqrt(D)).to(dtype)
    k = (torch.randn(*shp, D, generator=g) / math.sqrt(D)).to(dtype)
    v = torch.randn(*shp, DV, generator=g).to(dtype)
    gamma = 1.0 - torch.exp2(-5.0 - torch.arange(H, dtype=torch.float32))
    decay = gamma.view(1, H, 1).expand(B, H, S).contiguous()
    return q, k, v, decay


def mamba2_inputs(B, H, S, P, N, dtype=torch.bfloat16, seed=0):
    """x ~ N(0,1) [B,H,S,P]; Bm,Cm ~ N(0,1)/sqrt(N) [B,1,S,N] (single group);
    dt = softplus(N(0,1)-2) [B,H,S] fp32; A_h = -exp(U(0, log 16)) [1,H]."""
    g = _gen(seed)
    x = torch.randn(B, H, S, P, generator=g).to(dtype)
    Bm = (torch.randn(B, 1, S, N, generator=g) / math.sqrt(N)).to(dtype)
    Cm = (torch.randn(B, 1, S, N, generator=g) / math.sqrt(N)).to(dtype)
    dt = torch.nn.functional.softplus(torch.randn(B, H, S, generator=g) - 2.0)
    A = -torch.exp(torch.rand(1, H, generator=g) * math.log(16.0))
    return Cm, Bm, x, dt, A


def mla_inputs(B, HQ, SKV, D, DPE, dtype=torch.bfloat16, seed=0):
    """q [B,1,HQ,D], q_pe [B,1,HQ,DPE], kv [B,SKV,1,D], k_pe [B,SKV,1,DPE] ~ N(0,1)."""
    g = _gen(seed)
    q = torch.randn(B, 1, HQ, D, generator=g).to(dtype)
    q_pe = torch.randn(B, 1, HQ, DPE, generator=g).to(dtype)
    kv = torch.randn(B, SKV, 1, D, generator=g).to(dtype)
    k_pe = torch.randn(B, SKV, 1, DPE, generator=g).to(dtype)
    return q, q_pe, kv, k_pe
