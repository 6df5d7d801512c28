"""The reference's own test list (testing/test.py:54-63, `test_attention`), entry by entry at its shapes and dtypes, through
the operators built from the specs of `tests/specs.py` (the reference's examples restated) and called as its tests call them.
Forward against the oracle (the reference's PyTorch functions restated), and where the reference's test takes gradients
(`require_grad=True`: softmax, sigmoid, relu, mamba2, gated retention, retnet) the backward through autograd as well.  The
oracle gets whole tensors where that takes seconds and (batch, head) slices otherwise: heads are independent in every operator.
Tolerance atol 2e-2 / rtol 1e-2 with the allowances of the dedicated test files; the reference's own acceptance is looser
(1e-2 for softmax and MLA, 1e-1 for the others: testing/test.py:117,363,488,571,782,851)."""
import math

import pytest
import torch

import oracle
from oracle import inputs
import specs

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


def _grads(mod, tensors, dout, *custom):
    leaves = [t.cuda().requires_grad_(True) for t in tensors]
    o = mod(*leaves, *custom)
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    return o, [t.grad for t in leaves]


@pytest.mark.parametrize("B,H,S,D,DV", [(1, 16, 2048, 128, 128), (1, 16, 2048, 128, 256)])       # testing/test.py:54-55
def test_softmaxattention(B, H, S, D, DV):
    mod = specs.softmax_attention(B, H, S, D, DV, dtype=torch.float16)
    q, k, v = (t.half() for t in inputs.softmax_inputs(B, H, S, D, DV, seed=1))
    dout = torch.randn(B, S, H, DV, generator=torch.Generator().manual_seed(2)).half()
    o, grads = _grads(mod, (q, k, v), dout)
    ref = oracle.softmax_attention(q, k, v, causal=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=1e-2, atol=1e-2)                              # the reference's own tolerance (:117)
    for name, got, want in zip(("dq", "dk", "dv"), grads, oracle.attention_grads(oracle.softmax_attention, q, k, v, dout, causal=True)):
        oracle.assert_close(got.float().cpu(), want.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3, msg=name)


def test_softmaxattention_decode():                                                               # testing/test.py:56
    B, H, S, KV, D, DV = 8, 16, 1, 4096, 128, 128
    mod = specs.softmax_attention_decode(B, H, S, KV, D, DV)
    g = torch.Generator().manual_seed(3)
    q, k, v = torch.randn(B, S, H, D, generator=g).half(), torch.randn(B, KV, H, D, generator=g).half(), torch.randn(B, KV, H, DV, generator=g).half()
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(q, k, v, causal=False), rtol=1e-2, atol=1e-2)


def test_mamba2():                                                                                 # testing/test.py:57
    B, HQ, S, D, DV, HV = 1, 1, 2048, 128, 64, 80
    mod = specs.mamba2(B, HQ, S, D, DV, HK=1, HV=HV)
    Cm, Bm, x, dt, A = inputs.mamba2_inputs(B, HV, S, DV, D, seed=4)
    dout = (0.5 * torch.randn(B, HV, S, DV, generator=torch.Generator().manual_seed(5))).bfloat16()
    o, (dC, dB, dx) = _grads(mod, (Cm, Bm, x), dout, dt.cuda(), A.cuda(), dt.bfloat16().cuda())
    vs = dt.bfloat16().float()                      # (the operator multiplies x by the bf16 copy of dt, as the reference's fused v_mod does)
    oracle.assert_close(o.float().cpu(), oracle.linear_attention_chunked(Cm, Bm, x, dt * A.view(1, HV, 1), chunk=64, v_scale=vs), rtol=RTOL, atol=ATOL)
    ref2 = oracle.ssd_chunk_scan_combined(x.permute(0, 2, 1, 3), dt.permute(0, 2, 1), A[0], Bm.permute(0, 2, 1, 3), Cm.permute(0, 2, 1, 3),
                                          chunk_size=64).permute(0, 2, 1, 3)
    oracle.assert_close(o.float().cpu(), ref2, rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3)
    rq, rk, rv, _, _ = oracle.linear_attention_grads(Cm, Bm, x, dt * A.view(1, HV, 1), dout, v_scale=vs, chunk=256)
    for name, got, want in (("dC", dC, rq), ("dB", dB, rk), ("dx", dx, rv)):
        oracle.assert_close(got.float().cpu(), want.float(), rtol=1e-1, atol=1e-1, mismatch_ratio=1e-2, msg=name + " (reference acceptance)")
        oracle.assert_close(got.float().cpu(), want.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=5e-3, msg=name)


def test_gated_retention():                                                                        # testing/test.py:58
    B, H, S, D, DV = 8, 32, 2048, 256, 256
    mod = specs.gated_retention(B, H, S, D, DV)
    gen = torch.Generator().manual_seed(6)
    q, k = torch.randn(B, H, S, D, generator=gen).bfloat16(), torch.randn(B, H, S, D, generator=gen).bfloat16()
    v = torch.randn(B, H, S, DV, generator=gen).bfloat16()
    g = torch.nn.functional.logsigmoid(torch.randn(B, H, S, generator=gen)).clamp_min(-5)
    dout = (0.1 * torch.randn(B, H, S, DV, generator=gen)).bfloat16()
    gc = g.cuda().requires_grad_(True)
    o, (dq, dk, dv) = _grads(mod, (q, k, v), dout, gc)
    for b, h in ((0, 0), (3, 17), (7, 31)):
        cut = lambda t: t[b:b + 1, h:h + 1]
        ref = oracle.simple_gla_chunked(cut(q), cut(k), cut(v), cut(g))
        oracle.assert_close(cut(o).float().cpu(), ref, rtol=1e-1, atol=1e-1)                      # the reference's tolerance (:488)
        oracle.assert_close(cut(o).float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)   # (outputs of magnitude 10 - 30 in bf16)
        rq, rk, rv, rg, _ = oracle.linear_attention_grads(cut(q), cut(k), cut(v), cut(g), cut(dout), q_scale=D ** -0.5)
        for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
            oracle.assert_close(cut(got).float().cpu(), want.float(), rtol=1e-1, atol=1e-1, mismatch_ratio=1e-2, msg=f"{name} ({b},{h}) (reference acceptance)")
            oracle.assert_close(cut(got).float().cpu(), want.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=5e-3, msg=f"{name} ({b},{h})")
        assert float((cut(gc.grad).float().cpu() - rg.float()).abs().max()) <= max(0.03 * float(rg.abs().max()), 1e-2)


def test_sigmoid_attention():                                                                      # testing/test.py:59
    B, H, S, D, DV = 1, 32, 2048, 128, 128
    mod = specs.sigmoid_attention(B, H, S, D, DV, dtype=torch.float16)
    q, k, v = (t.half() for t in inputs.softmax_inputs(B, H, S, D, DV, seed=7))
    q = (q.float() * 0.1).half()                     # (scores of order 1: the spec has no 1 / sqrt(D), testing/test.py:545-550 scales its inputs)
    bias = torch.tensor([-math.log(S)])
    dout = (0.1 * torch.randn(B, S, H, DV, generator=torch.Generator().manual_seed(8))).half()    # scale of testing/test.py:571
    o, grads = _grads(mod, (q, k, v), dout, bias.cuda())
    ref = oracle.sigmoid_attention(q, k, v, float(bias), causal=True, softmax_scale=1.0)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)
    want = oracle.attention_grads(oracle.sigmoid_attention, q, k, v, dout, bias=float(bias), causal=True, softmax_scale=1.0)
    for name, got, w in zip(("dq", "dk", "dv"), grads, want):
        oracle.assert_close(got.float().cpu(), w.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=5e-3, msg=name)


def test_sparse_gqa_decode():                                                                      # testing/test.py:60
    B, H, G, S, D, DV, block = 8, 32, 8, 2048, 128, 128, 32
    mod = specs.sparse_gqa_decode(B, H, G, S, D, DV, block=block)
    g = torch.Generator().manual_seed(9)
    q, k, v = torch.randn(B, 1, H, D, generator=g).half(), torch.randn(B, S, G, D, generator=g).half(), torch.randn(B, S, G, DV, generator=g).half()
    lens = torch.full((B,), S, dtype=torch.int32)
    nblk = S // block
    bm = torch.zeros(B, G, nblk, dtype=torch.bool)                      # half of the blocks kept, chosen at random (testing/test.py:697-726)
    for b in range(B):
        for gi in range(G):
            bm[b, gi, torch.randperm(nblk, generator=g)[:nblk // 2]] = True
    o = mod(q.cuda(), k.cuda(), v.cuda(), block_mask=bm.cuda(), cache_seqlens=lens.cuda())
    torch.cuda.synchronize()
    assert o.shape == (B, H, DV)
    oracle.assert_close(o.float().cpu(), oracle.sparse_decode_attention(q, k, v, bm, lens, block_size=block), rtol=RTOL, atol=ATOL)


def test_retnet_recurrent():                                                                       # testing/test.py:61
    B, H, S, D, DV = 1, 32, 2048, 256, 512
    mod = specs.retnet_recurrent(B, H, S, D, DV)
    q = torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(10)).bfloat16()
    k = (0.1 * torch.randn(B, H, S, D, generator=torch.Generator().manual_seed(11))).bfloat16()   # keys at 0.1 as testing/test.py:750-756
    v = torch.randn(B, H, S, DV, generator=torch.Generator().manual_seed(12)).bfloat16()
    # heads 0 .. 31 with gamma_h = 1 - 2^(-5 - h): from head 19 on gamma rounds to 1 in fp32, as in the reference's own inputs
    decay = (1 - torch.exp2(-5 - torch.arange(H, dtype=torch.float32)))[None, :, None].expand(B, H, S).contiguous()
    dout = (0.1 * torch.randn(B, H, S, DV, generator=torch.Generator().manual_seed(13))).bfloat16()
    o, (dq, dk, dv) = _grads(mod, (q, k, v), dout, decay.cuda())
    for h in (0, 7, 31):
        cut = lambda t: t[:, h:h + 1]
        ref = oracle.linear_attention_chunked(cut(q), cut(k), cut(v), torch.log(cut(decay)), chunk=64, q_scale=D ** -0.5)
        oracle.assert_close(cut(o).float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3)
        rq, rk, rv, _, _ = oracle.linear_attention_grads(cut(q), cut(k), cut(v), torch.log(cut(decay)), cut(dout), q_scale=D ** -0.5)
        for name, got, want in (("dq", dq, rq), ("dk", dk, rk), ("dv", dv, rv)):
            oracle.assert_close(cut(got).float().cpu(), want.float(), rtol=1e-1, atol=1e-1, mismatch_ratio=1e-2, msg=f"{name} head {h} (reference acceptance)")
            oracle.assert_close(cut(got).float().cpu(), want.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=5e-3, msg=f"{name} head {h}")


def test_relu_attention():                                                                         # testing/test.py:62
    B, H, S, D, DV = 1, 6, 2048, 64, 64
    mod = specs.relu_attention(B, H, S, D, DV, dtype=torch.float16)
    q, k, v = (t.half() for t in inputs.softmax_inputs(B, H, S, D, DV, seed=14))
    k, v = (k.float() * 0.5).half(), (v.float() * 0.5).half()                                      # input scaling of testing/test.py:609-610
    dout = (0.1 * torch.randn(B, S, H, DV, generator=torch.Generator().manual_seed(15))).half()
    o, grads = _grads(mod, (q, k, v), dout)
    ref = oracle.relu_attention(q, k, v)
    oracle.assert_close(o.float().cpu(), ref, rtol=1e-1, atol=1e-1, mismatch_ratio=1e-3)           # the reference's acceptance (:623)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=2e-2)           # (un-normalised sums of ~1000 fp16 probabilities)
    for name, got, want in zip(("dq", "dk", "dv"), grads, oracle.attention_grads(oracle.relu_attention, q, k, v, dout)):
        oracle.assert_close(got.float().cpu(), want.float(), rtol=1e-1, atol=1e-1, mismatch_ratio=1e-3, msg=name + " (reference acceptance)")
        oracle.assert_close(got.float().cpu(), want.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-2, msg=name)


def test_mla_decode():                                                                             # testing/test.py:63
    B, HQ, SKV, D, DV = 8, 128, 2048, 576, 512
    mod = specs.mla_decode(B, HQ, SKV, D, DV, dtype=torch.float16)
    q, q_pe, kv, k_pe = inputs.mla_inputs(B, HQ, SKV, DV, D - DV, dtype=torch.float16, seed=16)
    o = mod(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda())
    torch.cuda.synchronize()
    assert o.shape == (B, 1, HQ, DV)
    oracle.assert_close(o.float().cpu(), oracle.mla_decode(q, q_pe, kv, k_pe), rtol=1e-2, atol=1e-2)   # the reference's tolerance (:851)
