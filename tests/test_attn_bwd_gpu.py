"""Parity of the parallel attention backward (dq, dk, dv through the C ABI and through autograd on
the AttentionEngine operators) with the gradient oracle (autograd over the fp64 restated forward, as
the reference's tests obtain their reference gradients: testing/test.py:119-125).  Tolerance atol 2e-2 /
rtol 1e-2 with a small allowance for the bf16/fp16 rounding of p and ds (the reference's own checks
use rtol = atol = 1e-1, :123-125, which is asserted with no allowance)."""
import math

import pytest
import torch

import oracle
from oracle import inputs
import specs

pytestmark = pytest.mark.gpu
ATOL, RTOL = 2e-2, 1e-2


def _hb():
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    return hb


def _check(got, ref, what):
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        a, b = a.float().cpu(), b.float()
        oracle.assert_close(a, b, rtol=1e-1, atol=1e-1, msg=f"{what}:{name} (reference acceptance)")
        oracle.assert_close(a, b, rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3, msg=f"{what}:{name}")


def _run(hb, family, q, k, v, dout, causal, scale, bias=0.0):
    fam = {"softmax": hb.MA_ATTN_SOFTMAX, "sigmoid": hb.MA_ATTN_SIGMOID, "relu": hb.MA_ATTN_RELU}[family]
    qc, kc, vc, dc = q.cuda(), k.cuda(), v.cuda(), dout.cuda()
    B, S, H, _ = q.shape
    lse = torch.empty(B, H, S, device="cuda") if family == "softmax" else None
    o = hb.attn_fwd(qc, kc, vc, family=fam, causal=causal, scale=scale, bias=bias, row_scale=lse)
    got = hb.attn_bwd(qc, kc, vc, o, dc, lse, family=fam, causal=causal, scale=scale, bias=bias)
    torch.cuda.synchronize()
    if family == "softmax":
        ref = oracle.attention_grads(oracle.softmax_attention, q, k, v, dout, causal=causal, softmax_scale=scale)
    elif family == "sigmoid":
        ref = oracle.attention_grads(oracle.sigmoid_attention, q, k, v, dout, bias=bias, causal=causal, softmax_scale=scale)
    else:
        ref = oracle.attention_grads(oracle.relu_attention, q, k, v, dout, softmax_scale=scale)
    return got, ref


@pytest.mark.parametrize("D,DV", [(128, 128), (64, 64), (128, 256), (256, 256), (256, 512), (192, 128)])
@pytest.mark.parametrize("B,H,Hkv,S,causal", [(1, 2, 2, 256, True), (2, 3, 3, 200, True), (1, 2, 2, 333, False), (1, 4, 2, 129, True), (1, 1, 1, 1, True)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_softmax_backward(D, DV, B, H, Hkv, S, causal, dtype):
    hb = _hb()
    g = torch.Generator().manual_seed(S + D)
    q = torch.randn(B, S, H, D, generator=g).to(dtype)
    k = torch.randn(B, S, Hkv, D, generator=g).to(dtype)
    v = torch.randn(B, S, Hkv, DV, generator=g).to(dtype)
    dout = torch.randn(B, S, H, DV, generator=g).to(dtype)
    print(f"softmax bwd D{D} DV{DV} B{B} H{H} Hkv{Hkv} S{S} causal={causal} {dtype}", flush=True)
    got, ref = _run(hb, "softmax", q, k, v, dout, causal, 1 / math.sqrt(D))
    _check(got, ref, "softmax")


@pytest.mark.parametrize("D,H,Hkv,S,causal", [(128, 4, 2, 1100, True), (64, 2, 2, 1060, True), (128, 2, 1, 1100, False)])
def test_softmax_backward_many_tiles(D, H, Hkv, S, causal):
    """Longer sequences: the tile ring of the dk / dv kernel wraps several times, a workgroup takes a pair of key blocks
    (an odd number of blocks leaves the middle one alone), the last tile and the last key block are partial."""
    hb = _hb()
    g = torch.Generator().manual_seed(S + D)
    q = torch.randn(1, S, H, D, generator=g).bfloat16()
    k = torch.randn(1, S, Hkv, D, generator=g).bfloat16()
    v = torch.randn(1, S, Hkv, D, generator=g).bfloat16()
    dout = torch.randn(1, S, H, D, generator=g).bfloat16()
    print(f"softmax bwd many tiles D{D} H{H} Hkv{Hkv} S{S} causal={causal}", flush=True)
    got, ref = _run(hb, "softmax", q, k, v, dout, causal, 1 / math.sqrt(D))
    _check(got, ref, "softmax")


@pytest.mark.parametrize("D,Sq,Skv", [(128, 200, 333), (128, 333, 200), (64, 70, 520), (128, 1, 300)])
def test_softmax_backward_cross_lengths(D, Sq, Skv):
    """Different numbers of queries and keys (no mask): the dq kernel walks Skv, the dk / dv kernel Sq."""
    hb = _hb()
    g = torch.Generator().manual_seed(Sq + Skv)
    q = torch.randn(2, Sq, 2, D, generator=g).bfloat16()
    k = torch.randn(2, Skv, 2, D, generator=g).bfloat16()
    v = torch.randn(2, Skv, 2, D, generator=g).bfloat16()
    dout = torch.randn(2, Sq, 2, D, generator=g).bfloat16()
    print(f"softmax bwd cross D{D} Sq{Sq} Skv{Skv}", flush=True)
    got, ref = _run(hb, "softmax", q, k, v, dout, False, 1 / math.sqrt(D))
    _check(got, ref, "softmax")


def test_backward_random_shapes():
    """A seeded sweep over batch, heads, group size, length, head size, family and mask."""
    hb = _hb()
    rng = torch.Generator().manual_seed(1234)
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=rng))
    for case in range(14):
        D = (64, 128)[ri(0, 1)]
        Hkv = ri(1, 3)
        H = Hkv * ri(1, 2)
        B, S = ri(1, 2), ri(1, 420)
        family = ("softmax", "softmax", "sigmoid", "relu")[ri(0, 3)]
        causal = bool(ri(0, 1)) and family != "relu"
        g = torch.Generator().manual_seed(case)
        q = torch.randn(B, S, H, D, generator=g).bfloat16()
        k = (0.7 * torch.randn(B, S, Hkv, D, generator=g)).bfloat16()
        v = (0.7 * torch.randn(B, S, Hkv, D, generator=g)).bfloat16()
        dout = (0.3 * torch.randn(B, S, H, D, generator=g)).bfloat16()
        print(f"random bwd case {case}: {family} B{B} H{H} Hkv{Hkv} S{S} D{D} causal={causal}", flush=True)
        got, ref = _run(hb, family, q, k, v, dout, causal, 1 / math.sqrt(D), bias=-1.0 if family == "sigmoid" else 0.0)
        for name, a, b in zip(("dq", "dk", "dv"), got, ref):
            oracle.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3, msg=f"case {case} {family}:{name}")


@pytest.mark.parametrize("family", ["sigmoid", "relu"])
@pytest.mark.parametrize("D,DV,S,causal", [(128, 128, 256, True), (64, 64, 200, False), (128, 128, 130, True)])
def test_sigmoid_relu_backward(family, D, DV, S, causal):
    hb = _hb()
    if family == "relu":
        causal = False
    B, H = 1, 2
    g = torch.Generator().manual_seed(S)
    q = torch.randn(B, S, H, D, generator=g).half()
    k = (0.5 * torch.randn(B, S, H, D, generator=g)).half()
    v = (0.5 * torch.randn(B, S, H, DV, generator=g)).half()
    dout = (0.1 * torch.randn(B, S, H, DV, generator=g)).half()      # scale of testing/test.py:571
    print(f"{family} bwd D{D} DV{DV} S{S} causal={causal}", flush=True)
    got, ref = _run(hb, family, q, k, v, dout, causal, 1 / math.sqrt(D), bias=-1.0 if family == "sigmoid" else 0.0)
    _check(got, ref, family)


def test_backward_mask_is_exact():
    """Gradients of rows / keys must not depend on anything behind the causal diagonal: poisoning q, dout
    of later rows leaves dk, dv contributions of earlier rows... checked as: truncating the sequence gives
    the same dq for the kept rows, bit for bit."""
    hb = _hb()
    B, H, S, D = 1, 2, 256, 128
    g = torch.Generator().manual_seed(1)
    q, k, v, dout = (torch.randn(B, S, H, D, generator=g).bfloat16().cuda() for _ in range(4))
    lse = torch.empty(B, H, S, device="cuda")
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=0.1, row_scale=lse)
    dq, dk, dv = hb.attn_bwd(q, k, v, o, dout, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=0.1)
    cut = 128
    q2, k2, v2, do2 = (t[:, :cut].contiguous() for t in (q, k, v, dout))
    lse2 = torch.empty(B, H, cut, device="cuda")
    o2 = hb.attn_fwd(q2, k2, v2, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=0.1, row_scale=lse2)
    dq2, _, _ = hb.attn_bwd(q2, k2, v2, o2, do2, lse2, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=0.1)
    torch.cuda.synchronize()
    assert torch.equal(dq[:, :cut], dq2)


def test_engine_backward_like_the_reference_test():
    """testing/test.py:107-125 at a reduced size: o.backward(do) on the operator built from the spec."""
    B, H, S, D = 1, 4, 512, 128
    mod = specs.softmax_attention(B, H, S, D, D, dtype=torch.float16)
    g = torch.Generator().manual_seed(2)
    q, k, v, dout = (torch.randn(B, S, H, D, generator=g).half() for _ in range(4))
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc)
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    ref = oracle.attention_grads(oracle.softmax_attention, q, k, v, dout, causal=True)
    _check((qc.grad, kc.grad, vc.grad), ref, "engine softmax")


def test_engine_deepseek_v2_lite_head_sizes():
    """The shape of the reference's own AMD benchmark, testing/benchmark_mi250.py:40-46 (causal softmax, 16 heads, Dqk 192,
    Dv 128, fp16, forward and o.backward(do)), at a reduced length: 192 is not a power of two, its rows live in 256-wide
    LDS rows whose last 64 columns are neither loaded nor read."""
    B, H, S, D, DV = 1, 16, 520, 192, 128
    mod = specs.softmax_attention(B, H, S, D, DV, dtype=torch.float16)
    g = torch.Generator().manual_seed(3)
    q, k = (torch.randn(B, S, H, D, generator=g).half() for _ in range(2))
    v, dout = (torch.randn(B, S, H, DV, generator=g).half() for _ in range(2))
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc)
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(q, k, v, causal=True), rtol=RTOL, atol=ATOL)
    ref = oracle.attention_grads(oracle.softmax_attention, q, k, v, dout, causal=True)
    _check((qc.grad, kc.grad, vc.grad), ref, "engine softmax 192/128")
    # columns 192.. of a wider tensor are not touched: q and k as slices of 256-wide storage filled with NaN behind them
    wide_q = torch.full((B, S, H, 256), float("nan"), dtype=torch.float16, device="cuda")
    wide_k = torch.full((B, S, H, 256), float("nan"), dtype=torch.float16, device="cuda")
    wide_q[..., :D], wide_k[..., :D] = q.cuda(), k.cuda()
    with torch.no_grad():
        o2 = mod(wide_q[..., :D], wide_k[..., :D], v.cuda())
    torch.cuda.synchronize()
    assert torch.equal(o2, o.detach())


def test_engine_sigmoid_backward_with_bias_tensor():
    """examples/sigmoid_attn.py operator: the bias is a custom input; its gradient slot is None (attn_tl.py:690-691)."""
    B, H, S, D = 1, 2, 256, 128
    mod = specs.sigmoid_attention(B, H, S, D, D, dtype=torch.float16)
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, S, H, D, generator=g).half()
    k = (0.5 * torch.randn(B, S, H, D, generator=g)).half()
    v = torch.randn(B, S, H, D, generator=g).half()
    dout = (0.1 * torch.randn(B, S, H, D, generator=g)).half()
    bias = torch.tensor([-2.0])
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc, bias.cuda())
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    ref = oracle.attention_grads(oracle.sigmoid_attention, q, k, v, dout, bias=-2.0, causal=True, softmax_scale=1.0)
    _check((qc.grad, kc.grad, vc.grad), ref, "engine sigmoid")


def test_engine_retention_backward_at_another_head_size():
    """The retention operator at 128 / 128 (not its own 256 / 512): o.backward(do) through the operator built from the spec."""
    B, H, S = 1, 2, 136
    mod = specs.retention_parallel(B, H, S, 128, 128)
    q, k, v, _ = inputs.retnet_inputs(B, H, S, 128, 128, seed=1, layout="bshd")
    q = (q.float() * 4.0).bfloat16()
    mask = oracle.retention_decay_mask(H, S).bfloat16()
    dout = (0.5 * torch.randn(B, S, H, 128, generator=torch.Generator().manual_seed(2))).bfloat16()
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc, mask.cuda())
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    ref = oracle.attention_grads(oracle.retention_parallel, q, k, v, dout, mask=mask, freeze_r=True)
    _check((qc.grad, kc.grad, vc.grad), ref, "engine retention 128/128")


def test_retention_backward_at_an_unbuilt_head_size_raises():
    """Head sizes without backward kernels (here 256 / 128): the forward runs, backward raises."""
    hb = _hb()
    B, H, S = 1, 2, 128
    q = torch.randn(B, S, H, 256, device="cuda").bfloat16()
    v = torch.randn(B, S, H, 128, device="cuda").bfloat16()
    mask = oracle.retention_decay_mask(H, S).bfloat16().cuda()
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_bwd(q, q, v, v, v, torch.ones(B, H, S, device="cuda"), family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask,
                    score_mask_t=mask.transpose(2, 3).contiguous())


MASKS = {
    "sliding_window": lambda b, h, q, k: (q >= k) & (q - k < 100),
    "prefix_lm": lambda b, h, q, k: (q >= k) | (k < 64),
    "per_head_window": lambda b, h, q, k: (q >= k) & (q - k < 32 * (h + 1)),
    "document": lambda b, h, q, k: (q >= k) & ((q // 150) == (k // 150)),
    "shifted_causal": lambda b, h, q, k: q - 128 >= k,          # rows 0..127 have no key at all
}


def _keep(mask_mod, B, H, Sq, Skv):
    return mask_mod(torch.arange(B).view(B, 1, 1, 1), torch.arange(H).view(1, H, 1, 1), torch.arange(Sq).view(1, 1, Sq, 1),
                    torch.arange(Skv).view(1, 1, 1, Skv)).expand(B, H, Sq, Skv)


@pytest.mark.parametrize("name", sorted(MASKS))
@pytest.mark.parametrize("family,D,S", [("softmax", 128, 300), ("softmax", 64, 512), ("sigmoid", 128, 260)])
def test_engine_backward_with_arbitrary_mask_mod(name, family, D, S):
    """Gradients under any mask_mod (the reference generates the mask_mod's code into its backward kernels,
    attn_tl.py:212-525): the element-wise keep mask in both orientations.  Oracle: autograd over
    oracle.masked_attention in fp64."""
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    B, H = 2, 3
    mask_mod = MASKS[name]
    scale = 1 / math.sqrt(D)
    if family == "softmax":
        meta = tuple(meta_tensor(B, H, S, D, dtype=torch.bfloat16) for _ in range(3))
        mod = AttentionEngine(meta, CustomIO(), lambda s_, io, b, h, q, k: s_ * scale, mask_mod, specs.OnlineSoftmax())
    else:
        mod = specs.sigmoid_attention(B, H, S, D, D, scale=scale, const_bias=-math.log(S), form="exp", mask_mod=mask_mod)
    assert mod.mask_kind in ("other", "other_bh")
    g = torch.Generator().manual_seed(S + D)
    q, k, v, dout = (torch.randn(B, S, H, D, generator=g).bfloat16() for _ in range(4))
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc)
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    keep = _keep(mask_mod, B, H, S, S)
    ref = oracle.attention_grads(oracle.masked_attention, q, k, v, dout, keep=keep, family=family, softmax_scale=scale, bias=-math.log(S))
    _check((qc.grad, kc.grad, vc.grad), ref, f"engine {family} {name}")
    # what is masked gets exactly no gradient: keys no query may see
    unseen = ~keep.any(dim=2)                                   # [B, H, Skv]
    if unseen.any():
        idx = unseen.permute(0, 2, 1).cuda()                    # [B, Skv, H]
        assert torch.count_nonzero(kc.grad[idx]) == 0 and torch.count_nonzero(vc.grad[idx]) == 0


@pytest.mark.parametrize("family,mask,D,S,bq,bk", [
    ("softmax", "causal", 128, 512, 128, 128), ("softmax", "none", 64, 384, 128, 32), ("softmax", "sliding_window", 128, 512, 128, 64),
    ("sigmoid", "causal", 128, 512, 256, 128), ("relu", "none", 128, 256, 128, 128)])
def test_engine_backward_with_external_block_mask(family, mask, D, S, bq, bk):
    """Gradients of a call that passes block_mask= at prefill shapes (the block-sparse operator of the reference has a
    forward only, blockattn_tl.py:123-234; here the caller's blocks, spread to elements and ANDed with the operator's
    mask, drive the same masked backward kernels).  Oracle: autograd over oracle.masked_attention in fp64."""
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    B, H = 2, 3
    scale = 1 / math.sqrt(D)
    mask_mod = specs.causal_mask if mask == "causal" else MASKS.get(mask)
    meta = tuple(meta_tensor(B, H, S, D, dtype=torch.bfloat16) for _ in range(3))
    score_mod = {"softmax": lambda s_, io, b, h, q, k: s_ * scale,
                 "sigmoid": lambda s_, io, b, h, q, k: 1 / (1 + (-(s_ * scale + (-math.log(S)))).exp()),
                 "relu": lambda s_, io, b, h, q, k: (s_ * scale).max(0)}[family]
    mod = AttentionEngine(meta, CustomIO(), score_mod, mask_mod, specs.OnlineSoftmax() if family == "softmax" else specs.OnlineIdentity(),
                          extern_block_mask=True)
    g = torch.Generator().manual_seed(S + bq + bk)
    q, k, v, dout = (torch.randn(B, S, H, D, generator=g).bfloat16() for _ in range(4))
    if family == "relu":                              # un-normalised sums: the input scale of the relu tests above
        k, v, dout = (0.5 * k.float()).bfloat16(), (0.5 * v.float()).bfloat16(), (0.1 * dout.float()).bfloat16()
    bm = (torch.rand(B, H, S // bq, S // bk, generator=g) < 0.6).to(torch.int8)
    bm[0, 0, 1] = 0                                   # a whole block of query rows without keys
    bm[1, 1, :, 0] = 0                                # a block of keys no query sees
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc, block_mask=bm.cuda())
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    keep = _keep(mask_mod, B, H, S, S) if mask_mod is not None else None
    ref = oracle.attention_grads(oracle.masked_attention, q, k, v, dout, keep=keep, block_mask=bm, family=family, softmax_scale=scale,
                                 bias=-math.log(S))
    _check((qc.grad, kc.grad, vc.grad), ref, f"block mask {family} {mask}")
    assert torch.count_nonzero(qc.grad[0, bq:2 * bq, 0]) == 0
    assert torch.count_nonzero(kc.grad[1, :bk, 1]) == 0 and torch.count_nonzero(vc.grad[1, :bk, 1]) == 0


@pytest.mark.parametrize("D,DV", [(128, 128), (192, 128), (128, 256)])
def test_masked_backward_through_the_c_abi_matches_causal(D, DV):
    """A lower-triangular keep mask through elem_mask / elem_mask_t gives the gradients of the causal flag (bit for bit:
    the same tiles, the same masked elements), grouped-query heads included; at the head sizes of the fused dk / dv kernel
    (128 / 128, 192 / 128: its masked form) and of the two-launch kernels (128 / 256)."""
    hb = _hb()
    B, H, Hkv, S = 1, 4, 2, 257
    g = torch.Generator().manual_seed(11)
    q = torch.randn(B, S, H, D, generator=g).bfloat16().cuda()
    k = torch.randn(B, S, Hkv, D, generator=g).bfloat16().cuda()
    v = torch.randn(B, S, Hkv, DV, generator=g).bfloat16().cuda()
    dout = torch.randn(B, S, H, DV, generator=g).bfloat16().cuda()
    lse = torch.empty(B, H, S, device="cuda")
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5, row_scale=lse)
    ref = hb.attn_bwd(q, k, v, o, dout, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5)
    sp = (S + 3) // 4 * 4
    buf = torch.zeros(1, 1, S, sp, dtype=torch.uint8, device="cuda")
    buf[0, 0, :, :S] = torch.tril(torch.ones(S, S, dtype=torch.uint8, device="cuda"))
    buf_t = torch.zeros(1, 1, S, sp, dtype=torch.uint8, device="cuda")
    buf_t[0, 0, :, :S] = torch.triu(torch.ones(S, S, dtype=torch.uint8, device="cuda"))
    got = hb.attn_bwd(q, k, v, o, dout, lse, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=D ** -0.5,
                      elem_mask=buf[..., :S], elem_mask_t=buf_t[..., :S])
    torch.cuda.synchronize()
    for a, b_ in zip(got, ref):
        assert torch.equal(a, b_)
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_bwd(q, k, v, o, dout, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=D ** -0.5,
                    elem_mask=buf[..., :S], elem_mask_t=buf_t[..., :S])


def test_backward_tile_skipping_changes_nothing():
    """Tile masks only skip tiles in which nothing is kept: the gradients are the same bits with and without them."""
    hb = _hb()
    B, H, S, D = 1, 2, 1024, 64
    g = torch.Generator().manual_seed(5)
    q, k, v, dout = (torch.randn(B, S, H, D, generator=g).bfloat16().cuda() for _ in range(4))
    i, j = torch.arange(S, device="cuda").view(S, 1), torch.arange(S, device="cuda").view(1, S)
    keep = ((i >= j) & (i - j < 300)).to(torch.uint8).view(1, 1, S, S)
    keep_t = keep.transpose(2, 3).contiguous()
    kbm = keep.view(1, 1, S // 128, 128, S // 32, 32).amax(dim=(3, 5)).contiguous()
    qbm = keep_t.view(1, 1, S // 128, 128, S // 32, 32).amax(dim=(3, 5)).contiguous()
    assert int(kbm.sum()) < kbm.numel() // 2 and int(qbm.sum()) < qbm.numel() // 2
    lse = torch.empty(B, H, S, device="cuda")
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=D ** -0.5, row_scale=lse, elem_mask=keep)
    kw = dict(family=hb.MA_ATTN_SOFTMAX, causal=False, scale=D ** -0.5, elem_mask=keep, elem_mask_t=keep_t)
    ref = hb.attn_bwd(q, k, v, o, dout, lse, **kw)
    got = hb.attn_bwd(q, k, v, o, dout, lse, kv_block_mask=kbm, q_block_mask=qbm, **kw)
    torch.cuda.synchronize()
    for a, b_ in zip(got, ref):
        assert torch.equal(a, b_)
    # entry 2 = the mask keeps every score of the tile (the element mask is then not read for it): the same bits again
    kbm2 = (kbm + keep.view(1, 1, S // 128, 128, S // 32, 32).amin(dim=(3, 5))).contiguous()
    qbm2 = (qbm + keep_t.view(1, 1, S // 128, 128, S // 32, 32).amin(dim=(3, 5))).contiguous()
    assert int((kbm2 == 2).sum()) > 0 and int((qbm2 == 2).sum()) > 0
    got2 = hb.attn_bwd(q, k, v, o, dout, lse, kv_block_mask=kbm2, q_block_mask=qbm2, **kw)
    torch.cuda.synchronize()
    for a, b_ in zip(got2, ref):
        assert torch.equal(a, b_)
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_bwd(q, k, v, o, dout, lse, kv_block_mask=kbm, q_block_mask=qbm, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=D ** -0.5)


def test_backward_full_size_properties():
    """Benchmark shape (B8 H32 S4096 D128, causal): (batch, head) slices against the gradient oracle, the last key's
    dk / dv come from the last query alone (closed form), and the gradients are linear in dout."""
    hb = _hb()
    B, H, S, D = 8, 32, 4096, 128
    scale = 1 / math.sqrt(D)
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v, dout = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(4))
    lse = torch.empty(B, H, S, device="cuda")
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale, row_scale=lse)
    dq, dk, dv = hb.attn_bwd(q, k, v, o, dout, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale)
    torch.cuda.synchronize()
    for t in (dq, dk, dv):
        assert torch.isfinite(t.float()).all()
    # the last key is seen by the last query only: dv[S-1] = p * dout[S-1], with p = exp(s * scale - lse)
    s_last = (q[:, -1].float() * k[:, -1].float()).sum(-1) * scale                      # [B, H]
    p_last = torch.exp(s_last - lse[:, :, -1])
    torch.testing.assert_close(dv[:, -1].float(), p_last.unsqueeze(-1) * dout[:, -1].float(), rtol=2e-2, atol=2e-2)
    for b, h in [(0, 0), (7, 31)]:
        sl = lambda t: t[b:b + 1, :, h:h + 1].cpu()
        ref = oracle.attention_grads(oracle.softmax_attention, sl(q), sl(k), sl(v), sl(dout), causal=True, softmax_scale=scale)
        _check((sl(dq), sl(dk), sl(dv)), ref, f"full size slice ({b},{h})")
    # linearity in dout (exact: a power of two commutes with every rounding on the way)
    dq2, dk2, dv2 = hb.attn_bwd(q, k, v, o, dout * 2, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale)
    torch.cuda.synchronize()
    assert torch.equal(dq2, dq * 2) and torch.equal(dk2, dk * 2) and torch.equal(dv2, dv * 2)


def test_deepseek_v2_lite_full_size():
    """The reference's AMD benchmark shape (testing/benchmark_mi250.py:40-46: B8 H16 S4096, Dqk 192 / Dv 128, fp16, causal),
    forward and backward through the C ABI: (batch, head) slices against the oracles, the closed form of the last key's dv,
    linearity in dout."""
    hb = _hb()
    B, H, S, D, DV = 8, 16, 4096, 192, 128
    scale = 1 / math.sqrt(D)
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k = (torch.randn(B, S, H, D, device="cuda", dtype=torch.float16, generator=g) for _ in range(2))
    v, dout = (torch.randn(B, S, H, DV, device="cuda", dtype=torch.float16, generator=g) for _ in range(2))
    lse = torch.empty(B, H, S, device="cuda")
    print("deepseek-v2-lite full size 192/128", flush=True)
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale, row_scale=lse)
    dq, dk, dv = hb.attn_bwd(q, k, v, o, dout, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale)
    torch.cuda.synchronize()
    for t in (o, dq, dk, dv):
        assert torch.isfinite(t.float()).all()
    s_last = (q[:, -1].float() * k[:, -1].float()).sum(-1) * scale
    p_last = torch.exp(s_last - lse[:, :, -1])
    torch.testing.assert_close(dv[:, -1].float(), p_last.unsqueeze(-1) * dout[:, -1].float(), rtol=2e-2, atol=2e-2)
    for b, h in [(0, 0), (7, 15), (3, 6)]:
        sl = lambda t: t[b:b + 1, :, h:h + 1].cpu()
        ref_o, ref_lse = oracle.softmax_attention(sl(q), sl(k), sl(v), causal=True, softmax_scale=scale, return_lse=True)
        oracle.assert_close(sl(o).float(), ref_o, rtol=RTOL, atol=ATOL)
        torch.testing.assert_close(lse[b:b + 1, h:h + 1].cpu(), ref_lse, rtol=1e-3, atol=1e-3)
        if (b, h) != (3, 6):
            ref = oracle.attention_grads(oracle.softmax_attention, sl(q), sl(k), sl(v), sl(dout), causal=True, softmax_scale=scale)
            _check((sl(dq), sl(dk), sl(dv)), ref, f"192/128 full size slice ({b},{h})")
    dq2, dk2, dv2 = hb.attn_bwd(q, k, v, o, dout * 2, lse, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale)
    torch.cuda.synchronize()
    # (fp16: not exact as in bf16 -- ds is rounded to the tensor dtype, and where it is subnormal in fp16 a doubling does not
    # commute with that rounding)
    for a2, a1 in ((dq2, dq), (dk2, dk), (dv2, dv)):
        torch.testing.assert_close(a2.float(), 2 * a1.float(), rtol=2e-2, atol=1e-3)
