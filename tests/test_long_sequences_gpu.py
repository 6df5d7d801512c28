"""Long sequences (32 K - 128 K tokens) through the parallel and the chunked operators.  The parallel family is held against
the definition evaluated in fp64 for single query rows (first, second, around the middle, on a 32 K boundary, last: a full
score matrix would not fit), its backward against two closed forms; the chunked family against the chunked oracle over the
whole sequence."""
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


def _hb():
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    return hb


@pytest.mark.parametrize("D,DV,B,H,S,dtype", [(128, 128, 2, 2, 131072, torch.bfloat16), (64, 64, 2, 4, 65536, torch.bfloat16),
                                               (192, 128, 1, 2, 65536, torch.float16), (256, 256, 1, 2, 32768, torch.bfloat16)])
def test_causal_softmax_long(D, DV, B, H, S, dtype):
    hb = _hb()
    g = torch.Generator(device="cuda").manual_seed(S)
    q = torch.randn(B, S, H, D, device="cuda", generator=g).to(dtype)
    k = (0.5 * torch.randn(B, S, H, D, device="cuda", generator=g)).to(dtype)
    v = (0.5 * torch.randn(B, S, H, DV, device="cuda", generator=g)).to(dtype)
    do = (0.5 * torch.randn(B, S, H, DV, device="cuda", generator=g)).to(dtype)
    lse = torch.full((B, H, S), float("nan"), device="cuda")
    scale = D ** -0.5
    print(f"long softmax D{D}/{DV} B{B} H{H} S{S} {dtype}", flush=True)
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale, row_scale=lse)
    dq, dk, dv = hb.attn_bwd(q, k, v, o, do, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale)
    torch.cuda.synchronize()
    for t in (o, dq, dk, dv, lse):
        assert torch.isfinite(t.float()).all()
    qc, kc, vc = q.cpu(), k.cpu(), v.cpu()
    for b, h, r in [(0, 0, 0), (0, H - 1, 1), (B - 1, 0, S // 2 + 17), (B - 1, H - 1, S - 1), (0, 0, S - 256), (0, H - 1, 32767), (0, 0, 32768 % S)]:
        s = (kc[b, :r + 1, h].double() @ qc[b, r, h].double()) * scale
        ref = torch.softmax(s, dim=0) @ vc[b, :r + 1, h].double()
        torch.testing.assert_close(o[b, r, h].double().cpu(), ref, rtol=1e-2, atol=2e-2, msg=f"row {(b, h, r)}")
        assert abs(float(lse[b, h, r]) - float(torch.logsumexp(s, 0))) < 1e-4, (b, h, r)
    # the first query sees one key: p = 1, ds = p (dp - sum p dp) = 0, so dq[0] = 0; the last key is seen by the last query only
    assert float(dq[:, 0].float().abs().max()) < 1e-6
    p_last = torch.exp((q[:, -1].float() * k[:, -1].float()).sum(-1) * scale - lse[:, :, -1])
    torch.testing.assert_close(dv[:, -1].float(), p_last.unsqueeze(-1) * do[:, -1].float(), rtol=2e-2, atol=1e-6)
    # key 0 is seen by every query: dv[0] = sum_i p_i0 do_i, with p_i0 = exp(s_i0 - lse_i)
    for b, h in [(0, 0), (B - 1, H - 1)]:
        p0 = torch.exp((q[b, :, h].float() @ k[b, 0, h].float()) * scale - lse[b, h])
        torch.testing.assert_close(dv[b, 0, h].float(), p0 @ do[b, :, h].float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("B,H,T,Dk,Dv", [(1, 2, 131072, 128, 128), (1, 1, 65536, 256, 512), (2, 1, 65536, 64, 64)])
def test_chunked_linear_long(B, H, T, Dk, Dv):
    hb = _hb()
    g = torch.Generator(device="cuda").manual_seed(T)
    q = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 4).bfloat16()
    k = (torch.randn(B, H, T, Dk, device="cuda", generator=g) / 4).bfloat16()
    v = torch.randn(B, H, T, Dv, device="cuda", generator=g).bfloat16()
    ld = torch.nn.functional.logsigmoid(torch.randn(B, H, T, device="cuda", generator=g) + 3.0)
    print(f"long linear B{B} H{H} T{T} Dk{Dk} Dv{Dv}", flush=True)
    o = hb.linear_fwd(q, k, v, ld, q_scale=Dk ** -0.5)
    torch.cuda.synchronize()
    ref = oracle.linear_attention_chunked(q.cpu(), k.cpu(), v.cpu(), ld.cpu(), chunk=64, q_scale=Dk ** -0.5)
    oracle.assert_close(o.float().cpu(), ref, rtol=1e-2, atol=2e-2)
