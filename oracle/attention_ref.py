"""CPU restatements of the parallel-attention and MLA-decode references.

Test infrastructure only (see the package docstring).  All functions take the
tensor layouts of the operators they check (BSHD for the parallel family),
up-cast to ``compute_dtype`` (fp32 by default, fp64 for pinning tests) and
loop over (batch, head) slices so the S x S score matrix of one head is the
largest temporary.
"""
from __future__ import annotations

import math
from typing import Optional

import torch


def _causal_keep(sq: int, skv: int, device) -> torch.Tensor:
    """keep[i, j] = (i >= j): the lower-triangular ``tril(ones)`` mask of
    testing/test.py:92-97 as a boolean matrix."""
    i = torch.arange(sq, device=device).unsqueeze(-1)
    j = torch.arange(skv, device=device).unsqueeze(0)
    return i >= j


def softmax_attention(q, k, v, causal: bool = True, softmax_scale: Optional[float] = None,
                      compute_dtype=torch.float32, return_lse: bool = False):
    """Softmax attention forward.  Follows testing/test.py:79-104 (and the
    identical attention_engine/benchmark/bench_utils.py:1347-1372): scores
    = q.k^T, masked with -inf above the diagonal, softmax(scores * scale), times
    v.  q [B,Sq,H,D], k [B,Skv,Hkv,D], v [B,Skv,Hkv,Dv] -> [B,Sq,H,Dv]; with Hkv < H
    query head h reads kv head h // (H // Hkv), the grouped-query layout of
    tl_template/attn/attn_gqa_tl.py:21-24, :80, :95 (all functions of this file).
    ``lse`` ([B,H,Sq], natural log, of the scaled scores) is the final row
    scale of examples/mha.py:65-71."""
    B, Sq, H, D = q.shape
    Skv, Dv = k.shape[1], v.shape[-1]
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    out = torch.empty(B, Sq, H, Dv, dtype=compute_dtype)
    lse = torch.empty(B, H, Sq, dtype=compute_dtype)
    keep = _causal_keep(Sq, Skv, q.device) if causal else None
    for b in range(B):
        for h in range(H):
            s = q[b, :, h].to(compute_dtype) @ k[b, :, h // (H // k.shape[2])].to(compute_dtype).T
            if keep is not None:
                s = s.masked_fill(~keep, float("-inf"))
            s = s * scale
            lse[b, h] = torch.logsumexp(s, dim=-1)
            out[b, :, h] = torch.softmax(s, dim=-1) @ v[b, :, h // (H // v.shape[2])].to(compute_dtype)
    return (out, lse) if return_lse else out


def sigmoid_attention(q, k, v, bias, causal: bool = True, softmax_scale: float = 1.0,
                      compute_dtype=torch.float32):
    """Sigmoid attention forward.  testing/test.py:519-543 is the unscaled
    form (bias added after the -inf masking, sigmoid written as
    (tanh(x/2)+1)/2); attention_engine/benchmark/bench_utils.py:806-832 is
    the scaled form (scores*scale + bias, then sigmoid).  ``bias`` is a python
    float or a 1-element tensor.  Masked positions contribute exactly 0."""
    B, Sq, H, D = q.shape
    Skv, Dv = k.shape[1], v.shape[-1]
    bias = float(bias.reshape(-1)[0]) if torch.is_tensor(bias) else float(bias)
    out = torch.empty(B, Sq, H, Dv, dtype=compute_dtype)
    keep = _causal_keep(Sq, Skv, q.device) if causal else None
    for b in range(B):
        for h in range(H):
            s = q[b, :, h].to(compute_dtype) @ k[b, :, h // (H // k.shape[2])].to(compute_dtype).T
            if keep is not None:
                s = s.masked_fill(~keep, float("-inf"))
            s = s * softmax_scale + bias
            p = (torch.tanh(s * 0.5) + 1.0) * 0.5
            out[b, :, h] = p @ v[b, :, h // (H // v.shape[2])].to(compute_dtype)
    return out


def relu_attention(q, k, v, softmax_scale: Optional[float] = None, compute_dtype=torch.float32):
    """ReLU attention forward, testing/test.py:599-604: relu(q.k^T / sqrt(D)) v,
    no mask, no normalisation."""
    B, Sq, H, D = q.shape
    Dv = v.shape[-1]
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    out = torch.empty(B, Sq, H, Dv, dtype=compute_dtype)
    for b in range(B):
        for h in range(H):
            s = q[b, :, h].to(compute_dtype) @ k[b, :, h // (H // k.shape[2])].to(compute_dtype).T
            out[b, :, h] = torch.relu(s * scale) @ v[b, :, h // (H // v.shape[2])].to(compute_dtype)
    return out


def retention_decay_mask(H: int, S: int, dtype=torch.float32) -> torch.Tensor:
    """[1,H,S,S] decay mask gamma_h^(i-j) * [i>=j] with gamma_h = 1 - 2^(-5-h),
    the RetNet head decays of testing/test.py:742-744 (there written in the
    log2 domain)."""
    g = 1.0 - torch.exp2(-5.0 - torch.arange(H, dtype=torch.float64))
    idx = torch.arange(S, dtype=torch.float64)
    diff = idx.unsqueeze(-1) - idx.unsqueeze(0)
    keep = diff >= 0
    m = torch.exp2(diff.clamp(min=0).unsqueeze(0) * torch.log2(g).view(H, 1, 1)) * keep
    return m.unsqueeze(0).to(dtype)


def retention_parallel(q, k, v, mask, compute_dtype=torch.float32, return_r: bool = False, freeze_r: bool = False):
    """Normalised parallel retention, attention_engine/benchmark/bench_utils.py:1158-1163
    (same as testing/benchmark_h100.py:808-813): qkm = (q.k^T) * mask,
    r = max(sum_j |qkm|, 1), o = (qkm / r) v.  q,k [B,S,H,D], v [B,S,H,Dv],
    mask [1 or B, H, S, S] -> [B,S,H,Dv].
    freeze_r: autograd sees r as a constant, which is the gradient the reference's operator defines
    (OnlineRetention.backward, examples/retention_parallel.py:82-86: dscores = dp / r, nothing flows through r)."""
    B, S, H, D = q.shape
    Dv = v.shape[-1]
    out = torch.empty(B, S, H, Dv, dtype=compute_dtype)
    r_out = torch.empty(B, H, S, dtype=compute_dtype)
    for b in range(B):
        mb = mask[b if mask.shape[0] > 1 else 0]
        for h in range(H):
            s = q[b, :, h].to(compute_dtype) @ k[b, :, h // (H // k.shape[2])].to(compute_dtype).T
            s = s * mb[h].to(compute_dtype)
            r = s.abs().sum(dim=-1, keepdim=True).clamp(min=1.0)
            if freeze_r:
                r = r.detach()
            r_out[b, h] = r.detach().squeeze(-1)
            out[b, :, h] = (s / r) @ v[b, :, h // (H // v.shape[2])].to(compute_dtype)
    return (out, r_out) if return_r else out


def mla_decode(q, q_pe, kv, k_pe, compute_dtype=torch.float32, return_lse: bool = False):
    """Absorbed MLA decode, testing/test.py:807-839 (same as
    attention_engine/core/template/tl_template/attn/mla_decode_tl.py:340-380):
    scores = (q.kv^T + q_pe.k_pe^T) / sqrt(d + d_pe), softmax over the cache,
    times kv.  q [B,1,Hq,d], q_pe [B,1,Hq,dpe], kv [B,Skv,Hkv,d],
    k_pe [B,Skv,Hkv,dpe] -> [B,1,Hq,d].  Query head h uses kv head
    h // (Hq // Hkv)."""
    B, _, Hq, d = q.shape
    dpe = q_pe.shape[-1]
    Hkv = kv.shape[2]
    group = Hq // Hkv
    scale = 1.0 / math.sqrt(d + dpe)
    out = torch.empty(B, 1, Hq, d, dtype=compute_dtype)
    lse = torch.empty(B, Hq, dtype=compute_dtype)
    for b in range(B):
        for g in range(Hkv):
            hs = slice(g * group, (g + 1) * group)
            qq = torch.cat([q[b, 0, hs], q_pe[b, 0, hs]], dim=-1).to(compute_dtype)
            kk = torch.cat([kv[b, :, g], k_pe[b, :, g]], dim=-1).to(compute_dtype)
            s = (qq @ kk.T) * scale
            lse[b, hs] = torch.logsumexp(s, dim=-1)
            out[b, 0, hs] = torch.softmax(s, dim=-1) @ kv[b, :, g].to(compute_dtype)
    return (out, lse) if return_lse else out


def attention_grads(forward, q, k, v, dout, **kwargs):
    """(dq, dk, dv) of ``sum(forward(q, k, v, **kwargs) * dout)`` by PyTorch autograd over the fp64
    restated forward, the way the reference's tests obtain reference gradients
    (testing/test.py:119-125: ``ref_o.backward(do)``)."""
    qd, kd, vd = (t.detach().to(torch.float64).requires_grad_(True) for t in (q, k, v))
    out = forward(qd, kd, vd, compute_dtype=torch.float64, **kwargs)
    out.backward(dout.to(torch.float64))
    return qd.grad, kd.grad, vd.grad


def sparse_decode_attention(q, k, v, block_mask=None, cache_seqlens=None, block_size: int = 32, compute_dtype=torch.float32):
    """Decode attention over a selected part of the cache, testing/test.py:654-693 (``ref_program_torch``):
    q [B,1,H,D], k [B,S,G,D], v [B,S,G,Dv]; keys in blocks of ``block_size`` whose ``block_mask[b, g, block]``
    is false, and keys at or beyond ``cache_seqlens[b]``, are set to -inf before softmax(scores / sqrt(D)).
    Query head h reads kv head h // (H // G).  Returns [B,H,Dv] (the query token squeezed, as there)."""
    B, _, H, D = q.shape
    S, G, Dv = k.shape[1], k.shape[2], v.shape[-1]
    out = torch.empty(B, H, Dv, dtype=compute_dtype)
    pos = torch.arange(S)
    for b in range(B):
        for h in range(H):
            g = h // (H // G)
            s = (k[b, :, g].to(compute_dtype) @ q[b, 0, h].to(compute_dtype)) / math.sqrt(D)
            keep = torch.ones(S, dtype=torch.bool)
            if block_mask is not None:
                keep &= block_mask[b, g].to(torch.bool).cpu()[pos // block_size]
            if cache_seqlens is not None:
                keep &= pos < int(cache_seqlens[b])
            s = s.masked_fill(~keep, float("-inf"))
            out[b, h] = torch.softmax(s, dim=-1) @ v[b, :, g].to(compute_dtype)
    return out


def masked_attention(q, k, v, keep=None, block_mask=None, family: str = "softmax", softmax_scale: Optional[float] = None,
                     bias: float = 0.0, compute_dtype=torch.float32):
    """Attention under an arbitrary element-wise mask and / or a block mask: the block-sparse prefill operator,
    tl_template/attn/blockattn_tl.py:123-234.  ``keep`` bool [1|B, 1|H, Sq, Skv] is the mask_mod evaluated densely
    (scores of dropped elements are -inf before the score function, :176-190); ``block_mask`` [1|B, 1|H, nq, nk]
    (non-zero = visit, :170) switches whole blocks of Sq/nq rows x Skv/nk keys off (:109-112).  family "softmax":
    softmax(scores * scale); "sigmoid": sigmoid(scores * scale + bias); "relu": max(scores * scale, 0); a dropped
    element contributes exactly 0 in each.  A row left without any key is all zeros (the epilogue is skipped when no
    block was visited, :225-227; a visited block whose elements are all dropped gives 0/0 there, defined as 0 here)."""
    B, Sq, H, D = q.shape
    Skv, Dv = k.shape[1], v.shape[-1]
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    out = torch.empty(B, Sq, H, Dv, dtype=compute_dtype)
    for b in range(B):
        for h in range(H):
            m = torch.ones(Sq, Skv, dtype=torch.bool)
            if keep is not None:
                m &= keep[b if keep.shape[0] > 1 else 0, h if keep.shape[1] > 1 else 0].to(torch.bool).cpu()
            if block_mask is not None:
                bm = block_mask[b if block_mask.shape[0] > 1 else 0, h if block_mask.shape[1] > 1 else 0].cpu() != 0
                nq, nk = bm.shape
                m &= bm.repeat_interleave(Sq // nq, dim=0).repeat_interleave(Skv // nk, dim=1)
            s = (q[b, :, h].to(compute_dtype) @ k[b, :, h // (H // k.shape[2])].to(compute_dtype).T) * scale
            if family == "softmax":
                p = torch.softmax(s.masked_fill(~m, float("-inf")), dim=-1)
                p = torch.where(m.any(dim=-1, keepdim=True), p, torch.zeros_like(p))
            elif family == "sigmoid":
                p = torch.sigmoid(s + bias) * m
            elif family == "relu":
                p = torch.relu(s) * m
            else:
                raise ValueError(family)
            out[b, :, h] = p @ v[b, :, h // (H // v.shape[2])].to(compute_dtype)
    return out


def biased_attention(q, k, v, add=None, causal: bool = False, family: str = "softmax", softmax_scale: Optional[float] = None,
                     bias: float = 0.0, softcap: Optional[float] = None, compute_dtype=torch.float32, return_lse: bool = False):
    """Attention whose score function adds score-free terms to the scaled score, the general form a ``score_mod`` with
    custom inputs takes: x = s * scale + bias + add[b, h, q, kv], then (``softcap``) x = softcap * tanh(x), then the row
    function of ``family`` ("softmax", "sigmoid", "relu").  ``add`` is anything that broadcasts to [B, H, Sq, Skv]: the
    reference's three custom-input classes (core/lower/lower.py:561-615: tensors without a seq_len_kv axis, [.., seq_len,
    seq_len_kv] tiles, seq_len_kv vectors) and index terms such as ALiBi's slope[h] * (kv_idx - q_idx) all reduce to it.
    The score_mod sits where the reference's kernel has it: after the -inf fill of masked scores and before the online
    row function (tl_template/attn/attn_tl.py:140-169), so a masked element contributes exactly 0.
    q,k [B,S,H,D], v [B,S,H,Dv] -> [B,Sq,H,Dv] (and the natural-log lse [B,H,Sq] for softmax)."""
    B, Sq, H, D = q.shape
    Skv, Dv = k.shape[1], v.shape[-1]
    scale = 1.0 / math.sqrt(D) if softmax_scale is None else softmax_scale
    out = torch.empty(B, Sq, H, Dv, dtype=compute_dtype)
    lse = torch.empty(B, H, Sq, dtype=compute_dtype)
    if add is not None:
        add = add.to(compute_dtype).expand(B, H, Sq, Skv)
    keep = _causal_keep(Sq, Skv, q.device) if causal else None
    for b in range(B):
        for h in range(H):
            x = (q[b, :, h].to(compute_dtype) @ k[b, :, h // (H // k.shape[2])].to(compute_dtype).T) * scale + bias
            if add is not None:
                x = x + add[b, h]
            if softcap is not None:
                x = softcap * torch.tanh(x)
            if keep is not None:
                x = x.masked_fill(~keep, float("-inf"))
            if family == "softmax":
                p = torch.softmax(x, dim=-1)
                lse[b, h] = torch.logsumexp(x, dim=-1)
            elif family == "sigmoid":
                p = torch.sigmoid(x)
            elif family == "relu":
                p = torch.relu(x).masked_fill(torch.isinf(x), 0.0)
            else:
                raise ValueError(family)
            out[b, :, h] = p @ v[b, :, h // (H // v.shape[2])].to(compute_dtype)
    return (out, lse) if return_lse and family == "softmax" else out


def paged_mla_decode(q, k_cache, block_table, cache_seqlens, head_dim_v: int = 512, compute_dtype=torch.float32):
    """flash_mla_with_kvcache semantics (cute_template_kvshared/flash_mla_interface.py:75-115) for one query
    token: q [B,1,Hq,d+dpe]; k_cache [pages, page_size, 1, d+dpe]; sequence b is the rows of pages
    block_table[b, 0], block_table[b, 1], ... truncated to cache_seqlens[b]; per sequence the absorbed MLA
    decode of ``mla_decode`` (scores over all d+dpe columns, values = the first d).  Returns (out [B,1,Hq,d],
    lse [B,Hq,1] natural log)."""
    B, _, Hq, Dfull = q.shape
    d = head_dim_v
    out = torch.empty(B, 1, Hq, d, dtype=compute_dtype)
    lse = torch.empty(B, Hq, 1, dtype=compute_dtype)
    for b in range(B):
        L = int(cache_seqlens[b])
        rows = k_cache[block_table[b].long()].reshape(-1, 1, Dfull)[:L]              # [L,1,Dfull]
        o, l = mla_decode(q[b:b + 1, :, :, :d], q[b:b + 1, :, :, d:], rows[None, :, :, :d], rows[None, :, :, d:],
                          compute_dtype=compute_dtype, return_lse=True)
        out[b], lse[b, :, 0] = o[0], l[0]
    return out, lse
