"""Parity of the HIP parallel-attention forward (through the C ABI) with the
CPU oracle on identical seeded inputs.  Tolerance: atol 2e-2, rtol 1e-2 on
fp32-accumulated bf16 results; masking checked exactly."""
import math

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


@pytest.mark.parametrize("B,H,S,causal", [
    (1, 2, 128, True), (2, 3, 256, True), (1, 2, 512, False), (1, 1, 64, True),
    (1, 2, 200, True), (1, 2, 333, False), (1, 1, 1, True), (1, 2, 129, True), (1, 1, 1000, False),
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_softmax_forward(B, H, S, causal, dtype):
    hb = _hb()
    D = 128
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, dtype=dtype, seed=S)
    ref, lse_ref = oracle.softmax_attention(q, k, v, causal=causal, return_lse=True)
    lse = torch.full((B, H, S), float("nan"), device="cuda")
    print(f"softmax B{B} H{H} S{S} causal={causal} {dtype}", flush=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=causal,
                    scale=1 / math.sqrt(D), row_scale=lse)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-4, atol=1e-4)


def test_softmax_full_size_property():
    """Full benchmark shape: compare a few (batch, head) slices against the oracle
    and check that lse is finite everywhere and the first row reproduces V
    (row 0 of a causal softmax attends only to kv 0)."""
    hb = _hb()
    B, H, S, D = 8, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(3))
    lse = torch.empty(B, H, S, device="cuda")
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=1 / math.sqrt(D), row_scale=lse)
    torch.cuda.synchronize()
    assert torch.isfinite(lse).all() and torch.isfinite(o.float()).all()
    assert torch.equal(o[:, 0], v[:, 0])
    for b, h in [(0, 0), (7, 31), (3, 17)]:
        ref = oracle.softmax_attention(q[b:b + 1, :, h:h + 1].cpu(), k[b:b + 1, :, h:h + 1].cpu(),
                                       v[b:b + 1, :, h:h + 1].cpu(), causal=True)
        oracle.assert_close(o[b:b + 1, :, h:h + 1].float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_sigmoid_full_size():
    """The sigmoid variant of the benchmark configuration at its full size (B8 H32 S4096 D128, causal,
    sigmoid(q.k * scale - log S)): three (batch, head) slices against the oracle at atol 2e-2 / rtol 1e-2, every
    output finite, and row 0 = sigmoid(score) * v[0] exactly as the oracle has it."""
    hb = _hb()
    B, H, S, D = 8, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(3))
    scale, bias = 1 / math.sqrt(D), -math.log(S)
    o = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SIGMOID, causal=True, scale=scale, bias=bias)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all()
    for b, h in [(0, 0), (7, 31), (4, 13)]:
        ref = oracle.sigmoid_attention(q[b:b + 1, :, h:h + 1].cpu(), k[b:b + 1, :, h:h + 1].cpu(), v[b:b + 1, :, h:h + 1].cpu(),
                                       bias, causal=True, softmax_scale=scale)
        oracle.assert_close(o[b:b + 1, :, h:h + 1].float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_causal_mask_is_exact():
    """Future keys must have exactly zero influence: poisoning k/v at positions
    > i must not change row i bit-for-bit."""
    hb = _hb()
    B, H, S, D = 1, 2, 256, 128
    q, k, v = (t.cuda() for t in inputs.softmax_inputs(B, H, S, D, D, seed=5))
    o1 = hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=0.1)
    cut = 100
    k2, v2 = k.clone(), v.clone()
    k2[:, cut:] = 1e4
    v2[:, cut:] = -1e4
    for fam in (hb.MA_ATTN_SOFTMAX, hb.MA_ATTN_SIGMOID, hb.MA_ATTN_RELU):
        oa = hb.attn_fwd(q, k, v, family=fam, causal=True, scale=0.1)
        ob = hb.attn_fwd(q, k2, v2, family=fam, causal=True, scale=0.1)
        torch.cuda.synchronize()
        assert torch.equal(oa[:, :cut], ob[:, :cut])
    assert torch.isfinite(o1.float()).all()


@pytest.mark.parametrize("B,H,S,causal", [(8, 16, 768, True), (3, 30, 1280, True), (2, 24, 1536, False), (16, 16, 768, True), (4, 8, 2304, True),
                                          (5, 8, 1792, True)])
def test_softmax_work_distribution(B, H, S, causal):
    """More work items than CUs, odd numbers of q blocks, (batch*head) counts that are and are not
    multiples of 8 and of 16 (with an even number of pairs per XCD a unit's two q blocks come from two pairs; B16: more
    than one such unit per workgroup; B5 H8: an odd number per XCD, both blocks from one pair): every item must be computed
    exactly once whatever the item -> workgroup mapping."""
    hb = _hb()
    D = 128
    g = torch.Generator(device="cuda").manual_seed(S)
    q, k, v = (torch.randn(B, S, H, D, device="cuda", dtype=torch.bfloat16, generator=g) for _ in range(3))
    o = torch.full((B, S, H, D), float("nan"), device="cuda", dtype=torch.bfloat16)
    lse = torch.full((B, H, S), float("nan"), device="cuda")
    print(f"work distribution B{B} H{H} S{S} causal={causal}", flush=True)
    hb.attn_fwd(q, k, v, family=hb.MA_ATTN_SOFTMAX, causal=causal, scale=1 / math.sqrt(D), out=o, row_scale=lse)
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    if causal:
        assert torch.equal(o[:, 0], v[:, 0])
    for b, h in [(0, 0), (B - 1, H - 1), (B // 2, H // 3)]:
        ref, lse_ref = oracle.softmax_attention(q[b:b + 1, :, h:h + 1].cpu(), k[b:b + 1, :, h:h + 1].cpu(),
                                                v[b:b + 1, :, h:h + 1].cpu(), causal=causal, return_lse=True)
        oracle.assert_close(o[b:b + 1, :, h:h + 1].float().cpu(), ref, rtol=RTOL, atol=ATOL)
        torch.testing.assert_close(lse[b:b + 1, h:h + 1].cpu(), lse_ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("B,H,S,causal", [(40, 16, 64, False), (40, 16, 96, True), (37, 9, 33, True), (40, 16, 128, False),
                                          (40, 16, 160, True), (20, 16, 288, False), (24, 16, 300, True)])
def test_softmax_many_short_items(B, H, S, causal):
    """Several short work items per workgroup: the first sub-tiles of an item are fetched by the last steps of the item
    before it (or, after an item of fewer than 4 sub-tiles, all at once), in every alignment of the ring; every row of
    every item is checked."""
    hb = _hb()
    D = 128
    g = torch.Generator().manual_seed(S + B)
    q, k, v = (torch.randn(B, S, H, D, generator=g).bfloat16() for _ in range(3))
    o = torch.full((B, S, H, D), float("nan"), device="cuda", dtype=torch.bfloat16)
    lse = torch.full((B, H, S), float("nan"), device="cuda")
    print(f"short items B{B} H{H} S{S} causal={causal}", flush=True)
    hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=causal, scale=1 / math.sqrt(D), out=o, row_scale=lse)
    torch.cuda.synchronize()
    ref, lse_ref = oracle.softmax_attention(q, k, v, causal=causal, return_lse=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_softmax_growing_and_jumping_scores(dtype):
    """Row maxima that keep growing along the kv axis (the reference point of the exponentials moves
    many times) and single keys whose score jumps by hundreds (no overflow, no loss of the rest)."""
    hb = _hb()
    B, H, S, D = 1, 2, 640, 128
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, dtype=dtype, seed=11)
    ramp = (1.0 + torch.arange(S, dtype=torch.float32) / 8.0).view(1, S, 1, 1)
    q = (q.float().abs() + 0.5).to(dtype)
    k = (k.float().abs() * ramp).to(dtype)                      # scores grow roughly linearly with the key index
    k[:, 333] = k[:, 333] * 6                                   # and one key towers over its neighbours
    for causal in (True, False):
        ref, lse_ref = oracle.softmax_attention(q, k, v, causal=causal, return_lse=True)
        lse = torch.full((B, H, S), float("nan"), device="cuda")
        print(f"growing scores causal={causal} {dtype}", flush=True)
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=causal, scale=1 / math.sqrt(D), row_scale=lse)
        torch.cuda.synchronize()
        assert torch.isfinite(o.float()).all()
        oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
        torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-4, atol=1e-3)


def test_softmax_cross_lengths():
    """Different query and key lengths without a mask."""
    hb = _hb()
    B, H, Sq, Skv, D = 2, 3, 300, 1000, 128
    q, _, _ = inputs.softmax_inputs(B, H, Sq, D, D, seed=21)
    _, k, v = inputs.softmax_inputs(B, H, Skv, D, D, seed=22)
    ref = oracle.softmax_attention(q, k, v, causal=False)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SOFTMAX, causal=False, scale=1 / math.sqrt(D))
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("S,causal,scale,bias", [(256, True, 1.0, -3.0), (192, False, 0.088, -5.5), (130, True, 0.088, 0.5)])
def test_sigmoid_forward(S, causal, scale, bias):
    hb = _hb()
    B, H, D = 1, 2, 128
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=7)
    if scale == 1.0:   # the unscaled spec is used with small-norm inputs
        q = (q.float() * 0.3).bfloat16()
    ref = oracle.sigmoid_attention(q, k, v, bias, causal=causal, softmax_scale=scale)
    bt = torch.tensor([bias], device="cuda")
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SIGMOID, causal=causal, scale=scale, bias_tensor=bt)
    o2 = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_SIGMOID, causal=causal, scale=scale, bias=bias)
    torch.cuda.synchronize()
    assert torch.equal(o, o2)
    # sums of S un-normalised probabilities: tolerance as a fraction of elements, like the reference's own check
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=2e-3)


def test_relu_forward():
    hb = _hb()
    B, H, S, D = 1, 2, 256, 128
    q, k, v = inputs.softmax_inputs(B, H, S, D, D, seed=9)
    k, v = (k.float() * 0.5).bfloat16(), (v.float() * 0.5).bfloat16()   # input scaling of testing/test.py:609-610
    ref = oracle.relu_attention(q, k, v)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RELU, causal=False, scale=1 / math.sqrt(D))
    torch.cuda.synchronize()
    # reference acceptance for this family: rtol=atol=1e-1, 1e-3 of elements may miss (testing/test.py:623)
    oracle.assert_close(o.float().cpu(), ref, rtol=1e-1, atol=1e-1, mismatch_ratio=1e-3)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3)


def test_rejects_bad_arguments():
    hb = _hb()
    q = torch.zeros(1, 64, 1, 128, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_fwd(q, q, q, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=-1.0)
    q96 = torch.zeros(1, 64, 1, 96, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(hb.MetaAttentionError) as ei:
        hb.attn_fwd(q96, q96, q96, family=hb.MA_ATTN_SOFTMAX, causal=True, scale=1.0)
    assert "no kernel" in str(ei.value)
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_fwd(q.cpu(), q.cpu(), q.cpu(), family=hb.MA_ATTN_SOFTMAX, causal=True, scale=1.0)
