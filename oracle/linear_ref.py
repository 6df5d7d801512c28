"""CPU restatements of the chunked linear / stateful attention references.

Test infrastructure only (see the package docstring).  Layout is BHSD as in
the linear operators (q [B,Hq,T,Dk], k [B,Hk,T,Dk], v [B,H,T,Dv]); the Mamba2
reference keeps its own (batch, seqlen, heads, dim) layout like the function
it restates.
"""
from __future__ import annotations

import math
from typing import Optional

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------
# RetNet (fixed per-head decay)
# --------------------------------------------------------------------------
def retnet_gammas(H: int, dtype=torch.float64) -> torch.Tensor:
    """gamma_h = 1 - 2^(-5-h) (testing/test.py:742, 754-755)."""
    return 1.0 - torch.exp2(-5.0 - torch.arange(H, dtype=dtype))


def retnet_quadratic(q, k, v, compute_dtype=torch.float32):
    """Un-normalised RetNet retention in its quadratic (decay-mask) form,
    testing/test.py:738-747: n[h,i,j] = gamma_h^(i-j) [i>=j] built in the
    log2 domain, s = (q d^-0.5) k^T * n, o = s v."""
    B, H, T, Dk = q.shape
    log2g = torch.log2(retnet_gammas(H, torch.float64))
    idx = torch.arange(T, dtype=torch.float64)
    diff = idx.unsqueeze(-1) - idx
    out = torch.empty(B, H, T, v.shape[-1], dtype=compute_dtype)
    for h in range(H):
        n = (torch.exp2(diff * log2g[h]) * (diff >= 0)).to(compute_dtype)
        for b in range(B):
            s = (q[b, h].to(compute_dtype) * Dk ** -0.5) @ k[b, h].to(compute_dtype).T
            out[b, h] = (s * n) @ v[b, h].to(compute_dtype)
    return out


def retnet_recurrence(q, k, v, compute_dtype=torch.float64):
    """Token-by-token form of the same operator: S_t = gamma S_{t-1} + k_t^T v_t,
    o_t = (q_t d^-0.5) S_t.  Independent of the quadratic form; used to pin it."""
    B, H, T, Dk = q.shape
    Dv = v.shape[-1]
    g = retnet_gammas(H, compute_dtype)
    out = torch.empty(B, H, T, Dv, dtype=compute_dtype)
    for b in range(B):
        for h in range(H):
            S = torch.zeros(Dk, Dv, dtype=compute_dtype)
            for t in range(T):
                S = g[h] * S + torch.outer(k[b, h, t].to(compute_dtype), v[b, h, t].to(compute_dtype))
                out[b, h, t] = (q[b, h, t].to(compute_dtype) * Dk ** -0.5) @ S
    return out


# --------------------------------------------------------------------------
# generic scalar-decay chunked linear attention (what the operator computes)
# --------------------------------------------------------------------------
def linear_attention_chunked(q, k, v, log_decay, chunk: int = 64, q_scale: float = 1.0,
                             v_scale: Optional[torch.Tensor] = None, compute_dtype=torch.float32):
    """Chunked evaluation of o_t = q_scale q_t sum_{s<=t} exp(G_t - G_s) k_s^T (v_s vs_s)
    with G the running sum of ``log_decay`` [B,H,T].  Follows the operator
    definition of tl_template/linear/linear_tl.py:1240-1269 (chunk-local cumsum
    :36-60, state recurrence :182-217, output :360-396).  q,k may have fewer
    heads than v (head h uses q/k head h // (H // Hq), :172, :351-352)."""
    B, H, T, Dv = v.shape
    Hq, Hk, Dk = q.shape[1], k.shape[1], q.shape[-1]
    assert T % chunk == 0
    out = torch.empty(B, H, T, Dv, dtype=compute_dtype)
    tri = torch.tril(torch.ones(chunk, chunk, dtype=torch.bool))
    for b in range(B):
        for h in range(H):
            qq = q[b, h // (H // Hq)].to(compute_dtype) * q_scale
            kk = k[b, h // (H // Hk)].to(compute_dtype)
            vv = v[b, h].to(compute_dtype)
            if v_scale is not None:
                vv = vv * v_scale[b, h].to(compute_dtype).unsqueeze(-1)
            gg = log_decay[b, h].to(compute_dtype)
            S = torch.zeros(Dk, Dv, dtype=compute_dtype)
            for c in range(T // chunk):
                sl = slice(c * chunk, (c + 1) * chunk)
                g = torch.cumsum(gg[sl], dim=0)
                qc, kc, vc = qq[sl], kk[sl], vv[sl]
                inter = (qc * torch.exp(g).unsqueeze(-1)) @ S
                w = torch.exp((g.unsqueeze(-1) - g.unsqueeze(0)).masked_fill(~tri, 0.0)) * tri
                out[b, h, sl] = inter + ((qc @ kc.T) * w) @ vc
                S = S * torch.exp(g[-1]) + (kc * torch.exp(g[-1] - g).unsqueeze(-1)).T @ vc
    return out


# --------------------------------------------------------------------------
# Mamba2 SSD
# --------------------------------------------------------------------------
def ssd_chunk_scan_combined(x, dt, A, Bm, Cm, chunk_size: int = 64, compute_dtype=torch.float32):
    """Restatement of ``ssd_chunk_scan_combined_ref`` and its three helpers
    (testing/test.py:206-343) for D=None, z=None, no dt bias/softplus.
    x [b,l,h,p], dt [b,l,h], A [h], Bm/Cm [b,l,g,n] -> [b,l,h,p].

    Steps as there: dA cumsum per chunk in high precision (:324-330); chunk
    states sum_l B_l decay_l dt_l x_l (:206-234); weighted cumulative state
    passing across chunks (:236-262); intra-chunk scores C.B^T * decay, causal,
    times dt, times x, plus C.prev_state * exp(dA_cumsum) (:264-309)."""
    b, l, h, p = x.shape
    g, n = Bm.shape[2], Bm.shape[3]
    assert l % chunk_size == 0
    c = l // chunk_size
    cd = compute_dtype
    x_ = x.to(cd).view(b, c, chunk_size, h, p)
    dt_ = dt.to(cd).permute(0, 2, 1).reshape(b, h, c, chunk_size)
    rep = h // g
    B_ = Bm.to(cd).repeat_interleave(rep, dim=2).view(b, c, chunk_size, h, n)
    C_ = Cm.to(cd).repeat_interleave(rep, dim=2).view(b, c, chunk_size, h, n)
    dA = dt_ * A.to(cd).view(1, h, 1, 1)
    dA_cs = torch.cumsum(dA, dim=-1)                               # [b,h,c,L]
    # 1. per-chunk states  [b,c,h,p,n]
    decay_states = torch.exp(dA_cs[..., -1:] - dA_cs)              # [b,h,c,L]
    w = (decay_states * dt_).permute(0, 2, 3, 1)                   # [b,c,L,h]
    states = torch.einsum("bclhn,bclh,bclhp->bchpn", B_, w, x_)
    # 2. state passing: state entering chunk z = sum_{c<z} exp(sum dA_chunk[c+1..z-1]) states[c]
    chunk_sum = dA_cs[..., -1]                                     # [b,h,c]
    cum = torch.cumsum(F.pad(chunk_sum, (1, 0)), dim=-1)           # [b,h,c+1]
    seg = cum.unsqueeze(-1) - cum.unsqueeze(-2)                    # [b,h,z,c']
    tri = torch.tril(torch.ones(c + 1, c + 1, dtype=torch.bool))
    decay_chunk = torch.exp(seg.masked_fill(~tri, 0.0)) * tri
    all_states = torch.cat([torch.zeros_like(states[:, :1]), states], dim=1)  # [b,c+1,h,p,n]
    passed = torch.einsum("bhzc,bchpn->bzhpn", decay_chunk, all_states)[:, :-1]
    # 3. outputs
    CB = torch.einsum("bclhn,bcshn->bchls", C_, B_)
    seg_in = dA_cs.unsqueeze(-1) - dA_cs.unsqueeze(-2)             # [b,h,c,L,S]
    tri_in = torch.tril(torch.ones(chunk_size, chunk_size, dtype=torch.bool))
    decay = (torch.exp(seg_in.masked_fill(~tri_in, 0.0)) * tri_in).permute(0, 2, 1, 3, 4)
    scores = CB * decay                                            # [b,c,h,L,S]
    out = torch.einsum("bchls,bhcs,bcshp->bclhp", scores, dt_, x_)
    state_decay_out = torch.exp(dA_cs).permute(0, 2, 3, 1).unsqueeze(-1)  # [b,c,L,h,1]
    out_prev = torch.einsum("bclhn,bchpn->bclhp", C_, passed) * state_decay_out
    return (out + out_prev).reshape(b, l, h, p)


def ssd_sequential(x, dt, A, Bm, Cm, compute_dtype=torch.float64):
    """Naive sequential state-space recurrence h_t = exp(dt_t A) h_{t-1} +
    dt_t B_t x_t^T, y_t = C_t h_t.  Independent of the chunked reference; used
    to pin it."""
    b, l, h, p = x.shape
    g, n = Bm.shape[2], Bm.shape[3]
    rep = h // g
    cd = compute_dtype
    out = torch.empty(b, l, h, p, dtype=cd)
    for bi in range(b):
        st = torch.zeros(h, n, p, dtype=cd)
        for t in range(l):
            dtt = dt[bi, t].to(cd)                                  # [h]
            Bt = Bm[bi, t].to(cd).repeat_interleave(rep, dim=0)     # [h,n]
            Ct = Cm[bi, t].to(cd).repeat_interleave(rep, dim=0)
            st = st * torch.exp(dtt * A.to(cd)).view(h, 1, 1) + \
                (dtt.view(h, 1) * Bt).unsqueeze(-1) * x[bi, t].to(cd).unsqueeze(1)
            out[bi, t] = torch.einsum("hn,hnp->hp", Ct, st)
    return out


# --------------------------------------------------------------------------
# gated retention / simple GLA (per-token log decay)
# --------------------------------------------------------------------------
def simple_gla_chunked(q, k, v, g, chunk_size: int = 64, scale: Optional[float] = None,
                       compute_dtype=torch.float32):
    """Restatement of ``naive_chunk_simple_gla`` (testing/test.py:436-481):
    q scaled by Dk^-0.5, per-chunk cumulative log decay, intra-chunk masked
    scores plus decayed inter-chunk state.  BHSD, g [B,H,T] (log space)."""
    scale = q.shape[-1] ** -0.5 if scale is None else scale
    return linear_attention_chunked(q, k, v, g, chunk=chunk_size, q_scale=scale,
                                    compute_dtype=compute_dtype)


def simple_gla_recurrence(q, k, v, g, scale: Optional[float] = None, compute_dtype=torch.float64):
    """Token recurrence S_t = exp(g_t) S_{t-1} + k_t^T v_t, o_t = scale q_t S_t."""
    B, H, T, Dk = q.shape
    Dv = v.shape[-1]
    scale = Dk ** -0.5 if scale is None else scale
    out = torch.empty(B, H, T, Dv, dtype=compute_dtype)
    for b in range(B):
        for h in range(H):
            S = torch.zeros(Dk, Dv, dtype=compute_dtype)
            for t in range(T):
                S = torch.exp(g[b, h, t].to(compute_dtype)) * S + \
                    torch.outer(k[b, h, t].to(compute_dtype), v[b, h, t].to(compute_dtype))
                out[b, h, t] = (q[b, h, t].to(compute_dtype) * scale) @ S
    return out


def linear_attention_grads(q, k, v, log_decay, dout, q_scale: float = 1.0, v_scale: Optional[torch.Tensor] = None, chunk: int = 16):
    """Gradients of sum(linear_attention_chunked(...) * dout) with respect to q, k, v, log_decay and
    v_scale (None without one), by PyTorch autograd over the fp64 chunked form - the way the
    reference's tests obtain reference gradients (testing/test.py:360-361, 483-484: ``o_ref.backward(do)``)."""
    T = q.shape[2]
    while T % chunk:
        chunk //= 2
    leaves = [t.detach().to(torch.float64).requires_grad_(True) for t in (q, k, v, log_decay)]
    vs = v_scale.detach().to(torch.float64).requires_grad_(True) if v_scale is not None else None
    out = linear_attention_chunked(*leaves, chunk=max(chunk, 1), q_scale=q_scale, v_scale=vs, compute_dtype=torch.float64)
    out.backward(dout.to(torch.float64))
    return tuple(t.grad for t in leaves) + ((vs.grad,) if vs is not None else (None,))
