"""The operators on tensors that are views: q, k, v cut out of one packed projection, a (batch, heads, seq, dim) storage seen
as (batch, seq, heads, dim), a fused MLA cache, expanded decay tensors.  The kernels read such views in place through their
strides; a view they cannot read (rows that do not start at 16-byte multiples) is copied once by the operator, and gradients
flow through the copy."""
import pytest
import torch

import oracle
from oracle import inputs
import specs

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


def test_parallel_operator_on_views():
    B, H, S, D = 2, 4, 300, 128
    mod = specs.softmax_attention(B, H, S, D, D)
    g = torch.Generator().manual_seed(0)
    qkv = torch.randn(B, S, 3, H, D, generator=g).bfloat16().cuda()          # packed projection
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    o = mod(q, k, v)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(q.cpu(), k.cpu(), v.cpu(), causal=True), rtol=RTOL, atol=ATOL)
    qt = torch.randn(B, H, S, D, generator=g).bfloat16().cuda().transpose(1, 2)   # BHSD storage seen as BSHD
    o = mod(qt, k, v)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(qt.cpu(), k.cpu(), v.cpu(), causal=True), rtol=RTOL, atol=ATOL)
    # gradients arrive in the packed tensor
    packed = qkv.clone().requires_grad_()
    dout = torch.randn(B, S, H, D, generator=g).bfloat16()
    mod(packed[:, :, 0], packed[:, :, 1], packed[:, :, 2]).backward(dout.cuda())
    torch.cuda.synchronize()
    ref = oracle.attention_grads(oracle.softmax_attention, q.cpu(), k.cpu(), v.cpu(), dout, causal=True)
    for i, name in enumerate(("dq", "dk", "dv")):
        oracle.assert_close(packed.grad[:, :, i].float().cpu(), ref[i].float(), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3, msg=name)
    # rows that start 8 bytes into a wider buffer: copied by the operator (the C ABI itself refuses them)
    wide = torch.randn(B, S, H, D + 8, generator=g).bfloat16().cuda().requires_grad_()
    o = mod(wide[..., 4:D + 4], k, v)
    o.sum().backward()
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(wide[..., 4:D + 4].detach().cpu(), k.cpu(), v.cpu(), causal=True), rtol=RTOL, atol=ATOL)
    assert torch.count_nonzero(wide.grad[..., :4]) == 0 and torch.count_nonzero(wide.grad[..., 4:D + 4]) > 0
    from metaattention_amd import hip_backend as hb
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_fwd(wide.detach()[..., 4:D + 4], k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5)


def test_linear_operator_on_views():
    g = torch.Generator().manual_seed(1)
    lin = specs.retnet_recurrent(1, 2, 160, 256, 512)
    q = torch.randn(1, 160, 2, 256, generator=g).bfloat16().cuda().transpose(1, 2)
    k = (0.1 * torch.randn(1, 160, 2, 256, generator=g)).bfloat16().cuda().transpose(1, 2)
    v = torch.randn(1, 160, 2, 512, generator=g).bfloat16().cuda().transpose(1, 2)
    decay = (1 - torch.exp2(-5 - torch.arange(2, dtype=torch.float32)))[None, :, None].expand(1, 2, 160).cuda()     # stride 0 along time
    o = lin(q, k, v, decay)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.retnet_quadratic(q.cpu(), k.cpu(), v.cpu()), rtol=RTOL, atol=ATOL)


def test_mla_operator_on_views():
    mla = specs.mla_decode(2, 16, 300, 576, 512)
    q, q_pe, kv, k_pe = (t.cuda() for t in inputs.mla_inputs(2, 16, 300, 512, 64, seed=5))
    ref = oracle.mla_decode(q.cpu(), q_pe.cpu(), kv.cpu(), k_pe.cpu())
    cache = torch.cat([kv, k_pe], dim=-1)                       # fused rows: two views with a 576-element row stride
    o = mla(q, q_pe, cache[..., :512], cache[..., 512:])
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    odd = torch.zeros(2, 300, 1, 580, dtype=torch.bfloat16, device="cuda")      # rows that start 4 bytes in: copied
    odd[..., 2:514], odd[..., 514:578] = kv, k_pe
    o = mla(q, q_pe, odd[..., 2:514], odd[..., 514:578])
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
