"""Parity of the parallel attention forward at the head sizes the 128/128 kernel does not take
(through the C ABI, against the CPU oracle): the shapes of the reference's own test list
(testing/test.py:54-63: softmax 128/256, relu 64/64) and their neighbours.  Tolerance atol 2e-2 /
rtol 1e-2; the un-normalised relu sums additionally at the reference's own acceptance."""
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


@pytest.mark.parametrize("D,DV", [(64, 64), (128, 256), (256, 256), (256, 512), (192, 128)])
@pytest.mark.parametrize("B,H,S,causal", [(1, 2, 256, True), (2, 3, 200, True), (1, 2, 333, False), (1, 1, 1, True), (1, 2, 129, True)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_softmax_other_head_sizes(D, DV, B, H, S, causal, dtype):
    hb = _hb()
    q, k, v = inputs.softmax_inputs(B, H, S, D, DV, dtype=dtype, seed=S + D)
    ref, lse_ref = oracle.softmax_attention(q, k, v, causal=causal, return_lse=True)
    lse = torch.full((B, H, S), float("nan"), device="cuda")
    print(f"softmax D{D} DV{DV} B{B} H{H} S{S} causal={causal} {dtype}", flush=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=causal, scale=1 / math.sqrt(D), row_scale=lse)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("D,DV", [(64, 64), (128, 256), (256, 512), (192, 128)])
@pytest.mark.parametrize("S,causal", [(256, True), (200, False), (130, True)])
def test_sigmoid_other_head_sizes(D, DV, S, causal):
    hb = _hb()
    B, H = 1, 2
    q, k, v = inputs.softmax_inputs(B, H, S, D, DV, dtype=torch.float16, seed=S + DV)
    bias = -math.log(S)
    ref = oracle.sigmoid_attention(q, k, v, bias, causal=causal, softmax_scale=1 / math.sqrt(D))
    print(f"sigmoid D{D} DV{DV} S{S} causal={causal}", flush=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SIGMOID, causal=causal, scale=1 / math.sqrt(D), bias=bias)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("B,H,S,D,DV", [(1, 6, 2048, 64, 64), (1, 2, 130, 64, 64), (1, 2, 256, 256, 512), (1, 2, 333, 192, 128)])
def test_relu_other_head_sizes(B, H, S, D, DV):
    """First case: the reference's own relu test (testing/test.py:62), fp16, inputs scaled as there (:609-610)."""
    hb = _hb()
    q, k, v = inputs.softmax_inputs(B, H, S, D, DV, dtype=torch.float16, seed=S)
    k, v = (k.float() * 0.5).half(), (v.float() * 0.5).half()
    ref = oracle.relu_attention(q, k, v)
    print(f"relu B{B} H{H} S{S} D{D} DV{DV}", flush=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RELU, causal=False, scale=1 / math.sqrt(D))
    torch.cuda.synchronize()
    # outputs are un-normalised sums over S keys: the reference accepts rtol=atol=1e-1 with 1e-3 of the elements off (:623)
    oracle.assert_close(o.float().cpu(), ref, rtol=1e-1, atol=1e-1, mismatch_ratio=1e-3)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3)


def test_reference_softmax_test_shape_128_256():
    """testing/test.py:55: B1 H16 S2048 D128 DV256, fp16, causal."""
    hb = _hb()
    B, H, S, D, DV = 1, 16, 2048, 128, 256
    q, k, v = inputs.softmax_inputs(B, H, S, D, DV, dtype=torch.float16, seed=55)
    ref = oracle.softmax_attention(q, k, v, causal=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=True, scale=1 / math.sqrt(D))
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_causal_mask_is_exact_other_head_sizes():
    """Poisoning keys and values behind the diagonal must not change a row bit for bit."""
    hb = _hb()
    for D, DV in ((64, 64), (128, 256), (256, 256), (192, 128)):
        B, H, S = 1, 2, 256
        q, k, v = (t.cuda() for t in inputs.softmax_inputs(B, H, S, D, DV, seed=D))
        cut = 100
        k2, v2 = k.clone(), v.clone()
        k2[:, cut:] = 1e4
        v2[:, cut:] = -1e4
        for fam in (hb.MA_ATTN_SOFTMAX, hb.MA_ATTN_SIGMOID, hb.MA_ATTN_RELU):
            oa = hb.attn_fwd(q, k, v, family=fam, causal=True, scale=0.1)
            ob = hb.attn_fwd(q, k2, v2, family=fam, causal=True, scale=0.1)
            torch.cuda.synchronize()
            assert torch.equal(oa[:, :cut], ob[:, :cut]), (D, DV, fam)


@pytest.mark.parametrize("D,DV", [(64, 64), (128, 256), (256, 256), (256, 512), (192, 128)])
def test_growing_scores_and_tile_size_independence(D, DV):
    """Row maxima that grow along the kv axis exercise the accumulator rescale (at Dv 512 the accumulators are rescaled
    in the MFMA accumulation registers); a constant key makes the output the running mean of v (closed form)."""
    hb = _hb()
    B, H, S = 1, 2, 300
    q, k, v = inputs.softmax_inputs(B, H, S, D, DV, seed=3)
    # positive q and k: the scores grow with the key index in every row (about 5 -> 30, the same at every head size), so the
    # reference of the exponentials moves every few tiles
    ramp = torch.linspace(0.2, 6.0, S).view(1, S, 1, 1) * (64 / D) ** 0.5
    q, k = q.abs(), (k.float().abs() * ramp).bfloat16()
    ref = oracle.softmax_attention(q, k, v, causal=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=True, scale=1 / math.sqrt(D))
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    kc = torch.ones_like(k)
    o2 = hb.attn_fwd(q.cuda(), kc.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=True, scale=1 / math.sqrt(D))
    mean = torch.cumsum(v.float(), dim=1) / torch.arange(1, S + 1).view(1, S, 1, 1)
    oracle.assert_close(o2.float().cpu(), mean, rtol=RTOL, atol=ATOL)


def test_engine_relu_64():
    """The relu operator built from the spec at the reference test's head size."""
    B, H, S, D = 1, 6, 512, 64
    mod = specs.relu_attention(B, H, S, D, D, dtype=torch.float16)
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, dtype=torch.float16, seed=8)
    k, v = (k.float() * 0.5).half(), (v.float() * 0.5).half()
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.relu_attention(q, k, v), rtol=1e-1, atol=1e-1, mismatch_ratio=1e-3)


@pytest.mark.parametrize("D,DV,H,Hkv", [(128, 128, 8, 2), (128, 128, 6, 1), (64, 64, 4, 2), (128, 256, 4, 1)])
@pytest.mark.parametrize("family", ["softmax", "sigmoid", "relu"])
def test_grouped_query_prefill(D, DV, H, Hkv, family):
    """k, v with fewer heads than q (attn_gqa_tl.py:21-24): both the 128/128 kernel and the others."""
    hb = _hb()
    B, S = 2, 300
    g = torch.Generator().manual_seed(D + H)
    q = torch.randn(B, S, H, D, generator=g).bfloat16()
    k = (0.5 * torch.randn(B, S, Hkv, D, generator=g)).bfloat16()
    v = (0.5 * torch.randn(B, S, Hkv, DV, generator=g)).bfloat16()
    scale = 1 / math.sqrt(D)
    print(f"gqa {family} D{D} DV{DV} H{H} Hkv{Hkv}", flush=True)
    if family == "softmax":
        ref = oracle.softmax_attention(q, k, v, causal=True)
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=True, scale=scale)
    elif family == "sigmoid":
        ref = oracle.sigmoid_attention(q, k, v, -3.0, causal=True, softmax_scale=scale)
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SIGMOID, causal=True, scale=scale, bias=-3.0)
    else:
        ref = oracle.relu_attention(q, k, v)
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RELU, causal=False, scale=scale)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3 if family == "relu" else 0.0)
    o_rep = hb.attn_fwd(q.cuda(), k.repeat_interleave(H // Hkv, dim=2).cuda(), v.repeat_interleave(H // Hkv, dim=2).cuda(),
                        family={"softmax": hb.MA_ATTN_SOFTMAX, "sigmoid": hb.MA_ATTN_SIGMOID, "relu": hb.MA_ATTN_RELU}[family],
                        causal=family != "relu", scale=scale, bias=-3.0 if family == "sigmoid" else 0.0)
    torch.cuda.synchronize()
    assert torch.equal(o, o_rep)     # the same arithmetic on the same values


def test_engine_grouped_query_softmax():
    """AttentionEngine with fewer kv heads (dispatch of attn_engine.py:327-343)."""
    B, H, Hkv, S, D = 1, 8, 2, 256, 128
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    meta = (meta_tensor(B, H, S, D, dtype=torch.float16), meta_tensor(B, Hkv, S, D, dtype=torch.float16), meta_tensor(B, Hkv, S, D, dtype=torch.float16))
    scale = 1 / math.sqrt(D)
    mod = AttentionEngine(meta, CustomIO(), lambda score, io, b, h, q_idx, kv_idx: score * scale, specs.causal_mask, specs.OnlineSoftmax())
    g = torch.Generator().manual_seed(0)
    q = torch.randn(B, S, H, D, generator=g).half()
    k = torch.randn(B, S, Hkv, D, generator=g).half()
    v = torch.randn(B, S, Hkv, D, generator=g).half()
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), oracle.softmax_attention(q, k, v, causal=True), rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("B,H,HKV,S,KV,D,DV", [(8, 16, 16, 1, 4096, 128, 128), (2, 32, 4, 1, 1000, 128, 128), (1, 4, 4, 3, 300, 64, 64),
                                             (8, 16, 16, 1, 2048, 192, 128)])   # (last: testing/benchmark_h100.py:63)
def test_engine_dense_decode(B, H, HKV, S, KV, D, DV):
    """Decode operators (first case: testing/test.py:56, reference function :131-148): a short query against a long cache,
    no mask, multi-head and grouped-query."""
    mod = specs.softmax_attention_decode(B, H, S, KV, D, DV, HKV=HKV)
    g = torch.Generator().manual_seed(KV)
    q = torch.randn(B, S, H, D, generator=g).half()
    k = torch.randn(B, KV, HKV, D, generator=g).half()
    v = torch.randn(B, KV, HKV, DV, generator=g).half()
    o = mod(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    assert o.shape == (B, S, H, DV)
    ref = oracle.softmax_attention(q, k, v, causal=False)
    oracle.assert_close(o.float().cpu(), ref, rtol=1e-2, atol=1e-2)      # the reference test's own tolerance (:156)


@pytest.mark.parametrize("B,H,G,S,D,DV,block", [(8, 32, 8, 2048, 128, 128, 32), (2, 8, 2, 500, 128, 128, 64), (3, 6, 6, 300, 64, 64, 32)])
def test_engine_sparse_gqa_decode(B, H, G, S, D, DV, block):
    """First case: testing/test.py:60 (block mask generated as there, :697-726, half of the blocks kept); the others add
    ragged cache lengths, a wider block and plain multi-head."""
    mod = specs.sparse_gqa_decode(B, H, G, S, D, DV, block=block)
    g = torch.Generator().manual_seed(S)
    q = torch.randn(B, 1, H, D, generator=g).half()
    k = torch.randn(B, S, G, D, generator=g).half()
    v = torch.randn(B, S, G, DV, generator=g).half()
    lens = torch.full((B,), S, dtype=torch.int32) if S == 2048 else torch.randint(1, S + 1, (B,), generator=g, dtype=torch.int32)
    nblk = (S + block - 1) // block
    bm = torch.zeros(B, G, nblk, dtype=torch.bool)
    for b in range(B):
        valid = (int(lens[b]) + block - 1) // block
        keep = max(1, math.ceil(int(lens[b]) * 0.5 / block))
        for gi in range(G):
            bm[b, gi, torch.randperm(valid, generator=g)[:keep]] = True
    o = mod(q.cuda(), k.cuda(), v.cuda(), block_mask=bm.cuda(), cache_seqlens=lens.cuda())
    torch.cuda.synchronize()
    assert o.shape == (B, H, DV)
    ref = oracle.sparse_decode_attention(q, k, v, bm, lens, block_size=block)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    # cache lengths alone (every block kept) through the same operator
    o2 = mod(q.cuda(), k.cuda(), v.cuda(), cache_seqlens=lens.cuda())
    torch.cuda.synchronize()
    oracle.assert_close(o2.float().cpu(), oracle.sparse_decode_attention(q, k, v, None, lens), rtol=RTOL, atol=ATOL)


def test_row_without_any_key_gives_zeros():
    hb = _hb()
    B, S, H, D = 1, 64, 1, 128
    q, k, v = (t.cuda() for t in inputs.softmax_inputs(B, H, S, D, D, seed=1))
    bm = torch.zeros(B, H, 2, dtype=torch.bool, device="cuda")
    lse = torch.empty(B, H, 1, device="cuda")
    o = hb.attn_fwd(q[:, :1].contiguous(), k, v, family=hb.MA_ATTN_SOFTMAX, causal=False, scale=0.1, kv_block_mask=bm, kv_block_size=32, row_scale=lse)
    torch.cuda.synchronize()
    assert float(o.float().abs().max()) == 0.0 and bool(torch.isinf(lse).all())


@pytest.mark.parametrize("D,DV", [(128, 128), (64, 64), (128, 256), (256, 256), (192, 128)])
@pytest.mark.parametrize("B,H,Hkv,Sq,Skv", [(8, 16, 16, 1, 4096), (2, 8, 2, 1, 1000), (1, 4, 4, 17, 700), (1, 2, 1, 32, 2048)])
def test_split_kv_decode_matches_unsplit(D, DV, B, H, Hkv, Sq, Skv):
    """Decode shapes through the split-KV path (workspace given: the default of the wrapper) and unsplit: both against
    the oracle, lse included, and against each other."""
    hb = _hb()
    g = torch.Generator().manual_seed(Skv + D)
    q = torch.randn(B, Sq, H, D, generator=g).half()
    k = torch.randn(B, Skv, Hkv, D, generator=g).half()
    v = torch.randn(B, Skv, Hkv, DV, generator=g).half()
    ref, lse_ref = oracle.softmax_attention(q, k, v, causal=False, return_lse=True)
    outs = []
    for split in (True, False):
        lse = torch.full((B, H, Sq), float("nan"), device="cuda")
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=False, scale=1 / math.sqrt(D), row_scale=lse,
                        split_kv=split)
        torch.cuda.synchronize()
        oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
        torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-3, atol=1e-3)
        outs.append(o)
    torch.testing.assert_close(outs[0].float(), outs[1].float(), rtol=1e-2, atol=2e-3)


def test_decode_workspace_sizes():
    hb = _hb()
    import ctypes
    p = hb.AttnParams()
    p.family, p.dtype, p.mask = hb.MA_ATTN_SOFTMAX, hb.MA_FP16, hb.MA_MASK_NONE
    p.batch, p.heads, p.seqlen_q, p.seqlen_kv, p.dim_qk, p.dim_v = 8, 16, 1, 4096, 128, 128
    lib = hb.load_library()
    need = lib.ma_attn_workspace_bytes(ctypes.byref(p))
    assert need == 8 * 8 * 16 * 1 * (128 * 2 + 4)          # 1024 / (8 * 16) = 8 splits
    p.mask = hb.MA_MASK_CAUSAL
    assert lib.ma_attn_workspace_bytes(ctypes.byref(p)) == 0
    p.mask, p.seqlen_q = hb.MA_MASK_NONE, 4096
    assert lib.ma_attn_workspace_bytes(ctypes.byref(p)) == 0


MASKS = {
    "sliding_window": lambda b, h, q, k: (q >= k) & (q - k < 100),
    "shifted_causal": lambda b, h, q, k: q - 128 >= k,                    # attention_engine/tests/test_blockmask.py:19-26
    "prefix_lm": lambda b, h, q, k: (q >= k) | (k < 64),
    "per_head_window": lambda b, h, q, k: (q >= k) & (q - k < 32 * (h + 1)),
    "document": lambda b, h, q, k: (q >= k) & ((q // 150) == (k // 150)),
}


@pytest.mark.parametrize("name", sorted(MASKS))
@pytest.mark.parametrize("D,S,family", [(128, 512, "softmax"), (64, 300, "softmax"), (128, 300, "sigmoid")])
def test_engine_arbitrary_mask_mod(name, D, S, family):
    """Any mask_mod (the reference generates its code into the block-sparse kernel, blockattn_tl.py:123-234): here through
    a dense keep mask + block mask.  Oracle: scores masked with -inf before the row function, rows without any key give 0."""
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    B, H = 2, 3
    mask_mod = MASKS[name]
    meta = tuple(meta_tensor(B, H, S, D, dtype=torch.bfloat16) for _ in range(3))
    scale = 1 / math.sqrt(D)
    if family == "softmax":
        mod = AttentionEngine(meta, CustomIO(), lambda s_, io, b, h, q, k: s_ * scale, mask_mod, specs.OnlineSoftmax())
    else:
        mod = specs.sigmoid_attention(B, H, S, D, D, scale=scale, const_bias=-math.log(S), form="exp", mask_mod=mask_mod)
    assert mod.mask_kind in ("other", "other_bh")
    g = torch.Generator().manual_seed(S)
    q = torch.randn(B, S, H, D, generator=g).bfloat16()
    k = torch.randn(B, S, H, D, generator=g).bfloat16()
    v = torch.randn(B, S, H, D, generator=g).bfloat16()
    o = mod(q.cuda(), k.cuda(), v.cuda())
    o2 = mod(q.cuda(), k.cuda(), v.cuda())          # second call re-uses the cached mask tensors
    torch.cuda.synchronize()
    assert torch.equal(o, o2)
    # the block mask attribute of the reference (attn_engine.py:394-397), at its default 128 x 128 blocks
    nb = (S + 127) // 128
    assert mod.block_mask is not None and mod.block_mask.shape[2:] == (nb, nb) and mod.block_mask.dtype == torch.int8
    bi, hi = torch.arange(B).view(B, 1, 1, 1), torch.arange(H).view(1, H, 1, 1)
    keep = mask_mod(bi, hi, torch.arange(S).view(1, 1, S, 1), torch.arange(S).view(1, 1, 1, S)).expand(B, H, S, S)
    ref = oracle.masked_attention(q, k, v, keep=keep, family=family, softmax_scale=scale, bias=-math.log(S))
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def _sparse_prefill_engine(family, causal, mask_mod, B, H, S, D, dtype=torch.bfloat16):
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    meta = tuple(meta_tensor(B, H, S, D, dtype=dtype) for _ in range(3))
    scale = 1 / math.sqrt(D)
    mm = mask_mod if mask_mod is not None else (specs.causal_mask if causal else None)
    if family == "softmax":
        return AttentionEngine(meta, CustomIO(), lambda s_, io, b, h, q, k: s_ * scale, mm, specs.OnlineSoftmax(), extern_block_mask=True)
    if family == "relu":
        return AttentionEngine(meta, CustomIO(), lambda s_, io, b, h, q, k: (s_ * scale).max(0), mm, specs.OnlineIdentity(),
                               extern_block_mask=True)
    return AttentionEngine(meta, CustomIO(), lambda s_, io, b, h, q, k: 1 / (1 + (-(s_ * scale + (-math.log(S)))).exp()), mm,
                           specs.OnlineIdentity(), extern_block_mask=True)


@pytest.mark.parametrize("family,mask,D,S,bq,bk", [
    ("softmax", "none", 128, 512, 128, 128),
    ("softmax", "causal", 128, 512, 128, 128),       # the reference's default block size (attn_engine.py:113)
    ("softmax", "causal", 64, 768, 256, 64),
    ("softmax", "sliding_window", 128, 512, 128, 32),
    ("sigmoid", "causal", 128, 512, 128, 64),
    ("relu", "none", 64, 256, 128, 32),
])
def test_engine_block_sparse_prefill(family, mask, D, S, bq, bk):
    """extern_block_mask=True at prefill shapes: mod(q, k, v, block_mask=[B, H, S/bq, S/bk]) visits only the kept blocks
    (blockattn_tl.py:123-234), on top of the mask_mod's element-wise mask; query blocks with no kept block give zeros."""
    B, H = 2, 3
    mask_mod = MASKS.get(mask)
    mod = _sparse_prefill_engine(family, mask == "causal", mask_mod, B, H, S, D)
    g = torch.Generator().manual_seed(S + bq + bk)
    q, k, v = (torch.randn(B, S, H, D, generator=g).bfloat16() for _ in range(3))
    bm = (torch.rand(B, H, S // bq, S // bk, generator=g) < 0.5).to(torch.int8)
    bm[0, 0, 1] = 0                                   # a whole block of query rows without keys
    bm[1, 2, 0] = 1
    o = mod(q.cuda(), k.cuda(), v.cuda(), block_mask=bm.cuda())
    torch.cuda.synchronize()
    keep = None
    if mask != "none":
        fn = mask_mod if mask_mod is not None else specs.causal_mask
        keep = fn(torch.arange(B).view(B, 1, 1, 1), torch.arange(H).view(1, H, 1, 1), torch.arange(S).view(1, 1, S, 1),
                  torch.arange(S).view(1, 1, 1, S)).expand(B, H, S, S)
    ref = oracle.masked_attention(q, k, v, keep=keep, block_mask=bm, family=family, softmax_scale=1 / math.sqrt(D), bias=-math.log(S))
    # (un-normalised relu sums: the rounding of the probabilities to bf16 alone is ~2.5e-2 rms at these sizes)
    ratio = 2e-2 if family == "relu" else 0.0
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=ratio)
    assert torch.count_nonzero(o[0, bq:2 * bq, 0]) == 0
    # a broadcast mask [1, 1, nq, nk], and the all-ones mask == the dense operator
    o1 = mod(q.cuda(), k.cuda(), v.cuda(), block_mask=bm[:1, :1].cuda())
    ref1 = oracle.masked_attention(q, k, v, keep=keep, block_mask=bm[:1, :1], family=family, softmax_scale=1 / math.sqrt(D), bias=-math.log(S))
    oracle.assert_close(o1.float().cpu(), ref1, rtol=RTOL, atol=ATOL, mismatch_ratio=ratio)


def test_blocks_kept_in_full_skip_the_element_mask():
    """Beside an element-wise mask, a block entry of 2 means "every score of the block is kept": the mask is not read for
    such blocks, and the output is the same bits as with entries of 1."""
    hb = _hb()
    B, H, S, D = 1, 2, 1024, 64
    g = torch.Generator().manual_seed(9)
    q, k, v = (torch.randn(B, S, H, D, generator=g).bfloat16().cuda() for _ in range(3))
    i, j = torch.arange(S, device="cuda").view(S, 1), torch.arange(S, device="cuda").view(1, S)
    keep = ((i >= j) & (i - j < 300)).to(torch.uint8).view(1, 1, S, S)
    tiles = keep.view(1, 1, S // 128, 128, S // 32, 32)
    any_, all_ = tiles.amax(dim=(3, 5)).contiguous(), tiles.amin(dim=(3, 5))
    assert int(all_.sum()) > 0
    kw = dict(family=hb.MA_ATTN_SOFTMAX, causal=False, scale=D ** -0.5, elem_mask=keep, kv_block_size=32)
    o1 = hb.attn_fwd(q, k, v, kv_block_mask=any_, **kw)
    o2 = hb.attn_fwd(q, k, v, kv_block_mask=(any_ + all_).contiguous(), **kw)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)


def test_block_sparse_prefill_rejects_odd_blocks():
    mod = _sparse_prefill_engine("softmax", True, None, 1, 2, 512, 128)
    q = torch.zeros(1, 512, 2, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError):
        mod(q, q, q, block_mask=torch.ones(1, 2, 8, 4, dtype=torch.int8, device="cuda"))      # 64-row query blocks
    with pytest.raises(ValueError):
        mod(q, q, q, block_mask=torch.ones(3, 2, 4, 4, dtype=torch.int8, device="cuda"))


def test_unsupported_head_size_is_an_error():
    hb = _hb()
    q = torch.zeros(1, 64, 1, 96, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(hb.MetaAttentionError) as ei:
        hb.attn_fwd(q, q, q, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=1.0)
    assert "no kernel" in str(ei.value)
