"""Parity of the HIP normalised parallel-retention forward (RETENTION family of
ma_attn_fwd) with the CPU oracle, directly and through the AttentionEngine operator."""
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


def _inputs(B, H, S, D, DV, seed, q_gain=4.0):
    q, k, v, _ = inputs.retnet_inputs(B, H, S, D, DV, seed=seed, layout="bshd")
    q = (q.float() * q_gain).bfloat16()       # row sums straddle the clamp at 1
    return q, k, v, oracle.retention_decay_mask(H, S).bfloat16()


@pytest.mark.parametrize("B,H,S,D,DV,causal", [
    (1, 2, 128, 256, 512, True), (2, 3, 200, 256, 512, True), (1, 2, 256, 128, 128, True),
    (1, 2, 132, 256, 512, False), (1, 1, 4, 256, 512, True), (1, 16, 512, 256, 512, True),
])
def test_retention_parallel(B, H, S, D, DV, causal):
    hb = _hb()
    q, k, v, mask = _inputs(B, H, S, D, DV, seed=S)
    ref, r_ref = oracle.retention_parallel(q, k, v, mask, return_r=True)
    assert (r_ref > 1).any()
    rs = torch.full((B, H, S), float("nan"), device="cuda")
    print(f"retention B{B} H{H} S{S} D{D} DV{DV} causal={causal}", flush=True)
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RETENTION, causal=causal, scale=1.0,
                    score_mask=mask.cuda(), row_scale=rs)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(rs.cpu(), r_ref, rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("B,H,S", [(1, 2, 128), (2, 3, 200), (1, 16, 700), (1, 1, 5)])
def test_retention_parallel_generated_decay_mask(B, H, S):
    """decay_gamma [H] instead of the multiplier tensor: the kernel generates gamma_h^(i - j) [i >= j] itself.  Checked
    against the oracle fed with that mask in fp32 (the tensor form rounds it to the tensor dtype first), and against the
    tensor path of the same kernel within the rounding of the bf16 mask."""
    hb = _hb()
    D, DV = 256, 512
    q, k, v, mask_bf16 = _inputs(B, H, S, D, DV, seed=S + 1)
    mask = oracle.retention_decay_mask(H, S)                    # fp32
    gamma = (1.0 - torch.exp2(-5.0 - torch.arange(H, dtype=torch.float64))).float()
    ref, r_ref = oracle.retention_parallel(q, k, v, mask, return_r=True)
    rs = torch.full((B, H, S), float("nan"), device="cuda")
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, decay_gamma=gamma.cuda(),
                    row_scale=rs)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(rs.cpu(), r_ref, rtol=1e-3, atol=1e-3)
    if S % 4 == 0:   # (the tensor form wants 8-byte aligned mask rows)
        o_t = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask_bf16.cuda())
        torch.cuda.synchronize()
        oracle.assert_close(o.float().cpu(), o_t.float().cpu(), rtol=2 * RTOL, atol=2 * ATOL)
    with pytest.raises(hb.MetaAttentionError):   # the generated mask is lower triangular: it goes with the causal structural mask
        hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RETENTION, causal=False, scale=1.0, decay_gamma=gamma.cuda())


def test_clamp_branch_leaves_rows_unnormalised():
    """Tiny scores: every row sum is below 1, r = 1 everywhere, o = (qk * M) v exactly as un-normalised retention."""
    hb = _hb()
    B, H, S, D, DV = 1, 2, 128, 256, 512
    q, k, v, mask = _inputs(B, H, S, D, DV, seed=1, q_gain=0.05)
    ref, r_ref = oracle.retention_parallel(q, k, v, mask, return_r=True)
    assert float(r_ref.max()) == 1.0
    rs = torch.empty(B, H, S, device="cuda")
    o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask.cuda(), row_scale=rs)
    torch.cuda.synchronize()
    assert torch.equal(rs.cpu(), torch.ones(B, H, S))
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)


def test_engine_retention_parallel():
    """mod(q, k, v, mask) as in testing/benchmark_h100.py:794-801."""
    B, H, S, D, DV = 2, 4, 256, 256, 512
    mod = specs.retention_parallel(B, H, S, D, DV)
    q, k, v, mask = _inputs(B, H, S, D, DV, seed=2)
    o = mod(q.cuda(), k.cuda(), v.cuda(), mask.cuda())
    torch.cuda.synchronize()
    ref, r_ref = oracle.retention_parallel(q, k, v, mask, return_r=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(mod.final_rowscales.cpu(), r_ref, rtol=1e-3, atol=1e-3)


def test_engine_takes_the_generated_mask_path_only_for_exponential_decay_masks():
    """The operator verifies on the device, once per mask tensor, whether the multiplier is gamma_h^(i - j) below the
    diagonal; only then does the kernel generate it (examples/retention_parallel.py:25-111 builds such a mask).  Any other
    multiplier -- here the same mask with one entry changed in place -- runs through the tensor path, bit for bit."""
    hb = _hb()
    B, H, S, D, DV = 2, 4, 256, 256, 512
    mod = specs.retention_parallel(B, H, S, D, DV)
    q, k, v, mask = _inputs(B, H, S, D, DV, seed=4)
    qc, kc, vc, mc = q.cuda(), k.cuda(), v.cuda(), mask.cuda()
    with torch.no_grad():
        o = mod(qc, kc, vc, mc)
    torch.cuda.synchronize()
    found = [g for _, _, g in mod._gamma_cache if g is not None]
    assert len(found) == 1
    gamma_ref = 1.0 - torch.exp2(-5.0 - torch.arange(H, dtype=torch.float64))
    torch.testing.assert_close(found[0].cpu().double(), gamma_ref, rtol=2e-5, atol=0)
    ref, r_ref = oracle.retention_parallel(q, k, v, mask, return_r=True)
    oracle.assert_close(o.float().cpu(), ref, rtol=RTOL, atol=ATOL)
    torch.testing.assert_close(mod.final_rowscales.cpu(), r_ref, rtol=2e-3, atol=2e-3)   # (fp32 factors against the rounded tensor's)
    # not an exponential decay any more: the tensor is read
    mc[0, 1, 200, 17] = 0.5
    with torch.no_grad():
        o2 = mod(qc, kc, vc, mc)
    direct = hb.attn_fwd(qc, kc, vc, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mc)
    torch.cuda.synchronize()
    assert any(g is None for _, _, g in mod._gamma_cache)
    assert torch.equal(o2, direct)
    # another tensor object is looked at afresh, whatever address it lives at (a new mask may sit in recycled memory)
    del mc
    other = torch.tril(torch.rand(1, H, S, S, device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))).bfloat16()
    with torch.no_grad():
        o4 = mod(qc, kc, vc, other)
    torch.cuda.synchronize()
    assert torch.equal(o4, hb.attn_fwd(qc, kc, vc, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=other))
    # gradients are asked for: the tensor path (the backward kernels read the tensor)
    mask2 = mask.cuda()
    qg = qc.clone().requires_grad_(True)
    o3 = mod(qg, kc, vc, mask2)
    torch.cuda.synchronize()
    assert torch.equal(o3.detach(), hb.attn_fwd(qc, kc, vc, family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, score_mask=mask2))


def _check_grads(got, ref, what):
    for name, a, b in zip(("dq", "dk", "dv"), got, ref):
        oracle.assert_close(a.float().cpu(), b.float(), rtol=RTOL, atol=ATOL, mismatch_ratio=1e-3, msg=f"{what}:{name}")


@pytest.mark.parametrize("B,H,S,causal,dtype,D,DV", [(1, 2, 128, True, torch.bfloat16, 256, 512), (2, 3, 200, True, torch.bfloat16, 256, 512),
                                                     (1, 2, 132, False, torch.bfloat16, 256, 512), (1, 1, 4, True, torch.bfloat16, 256, 512),
                                                     (1, 2, 260, True, torch.float16, 256, 512),
                                                     (1, 2, 200, True, torch.bfloat16, 128, 128), (2, 2, 136, True, torch.bfloat16, 64, 64),
                                                     (1, 2, 160, False, torch.bfloat16, 128, 256), (1, 2, 144, True, torch.bfloat16, 256, 256)])
def test_retention_backward(B, H, S, causal, dtype, D, DV):
    """dq, dk, dv of the retention operator through the C ABI: the row scale r of the forward pass is a constant of the
    backward (examples/retention_parallel.py:82-86).  Oracle: autograd over oracle.retention_parallel(freeze_r=True)
    in fp64."""
    hb = _hb()
    q, k, v, mask = _inputs(B, H, S, D, DV, seed=S)
    q, k, v, mask = (t.to(dtype) for t in (q, k, v, mask))
    dout = (0.5 * torch.randn(B, S, H, DV, generator=torch.Generator().manual_seed(S))).to(dtype)
    if not causal:
        mask = (mask.float() + mask.float().transpose(2, 3)).to(dtype)     # a full multiplier: decay on both sides of the diagonal
    qc, kc, vc, mc = q.cuda(), k.cuda(), v.cuda(), mask.cuda()
    rs = torch.empty(B, H, S, device="cuda")
    print(f"retention bwd B{B} H{H} S{S} D{D} DV{DV} causal={causal} {dtype}", flush=True)
    o = hb.attn_fwd(qc, kc, vc, family=hb.MA_ATTN_RETENTION, causal=causal, scale=1.0, score_mask=mc, row_scale=rs)
    got = hb.attn_bwd(qc, kc, vc, o, dout.cuda(), rs, family=hb.MA_ATTN_RETENTION, causal=causal, scale=1.0,
                      score_mask=mc, score_mask_t=mc.transpose(2, 3).contiguous())
    torch.cuda.synchronize()
    assert (rs > 1).any()
    ref = oracle.attention_grads(oracle.retention_parallel, q, k, v, dout, mask=mask, freeze_r=True)
    _check_grads(got, ref, "retention")


def test_engine_retention_backward():
    """o.backward(do) on the operator built from the spec (testing/test.py:107-125 does this for the softmax operator)."""
    B, H, S, D, DV = 2, 4, 256, 256, 512
    mod = specs.retention_parallel(B, H, S, D, DV)
    q, k, v, mask = _inputs(B, H, S, D, DV, seed=5)
    dout = (0.5 * torch.randn(B, S, H, DV, generator=torch.Generator().manual_seed(5))).bfloat16()
    qc, kc, vc = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = mod(qc, kc, vc, mask.cuda())
    o.backward(dout.cuda())
    torch.cuda.synchronize()
    ref = oracle.attention_grads(oracle.retention_parallel, q, k, v, dout, mask=mask, freeze_r=True)
    _check_grads((qc.grad, kc.grad, vc.grad), ref, "engine retention")


def test_retention_backward_needs_its_inputs():
    hb = _hb()
    q = torch.zeros(1, 64, 1, 256, device="cuda", dtype=torch.bfloat16)
    v = torch.zeros(1, 64, 1, 512, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(hb.MetaAttentionError):
        hb.attn_bwd(q, q, v, v, v, torch.ones(1, 1, 64, device="cuda"), family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0)


def test_parallel_and_chunked_forms_agree_at_full_size():
    """B=8 H=16 S=2048 Dqk=256 Dv=512: the parallel operator (mask = gamma^(i-j)) times its
    row scale r is the un-normalised retention the chunked operator computes."""
    hb = _hb()
    B, H, S, D, DV = 8, 16, 2048, 256, 512
    q, k, v, decay = (t.cuda() for t in inputs.retnet_inputs(B, H, S, D, DV, seed=0))          # BHSD
    qs = (q.float() * 0.05).bfloat16()
    mask = oracle.retention_decay_mask(H, S).bfloat16().cuda()
    rs = torch.empty(B, H, S, device="cuda")
    o_par = hb.attn_fwd(qs.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), family=hb.MA_ATTN_RETENTION, causal=True,
                        scale=1.0, score_mask=mask, row_scale=rs)
    o_chk = hb.linear_fwd(qs, k, v, torch.log(decay), q_scale=1.0)
    torch.cuda.synchronize()
    assert float(rs.min()) == 1.0 and float(rs.max()) > 1.0
    # the mask tensor is bf16-rounded gamma^(i-j); the chunked form uses fp32 decays
    torch.testing.assert_close(o_par.transpose(1, 2).float() * rs.unsqueeze(-1), o_chk.float(), rtol=3e-2, atol=4e-3)


@pytest.mark.parametrize("generated", [False, True], ids=["mask_tensor", "decay_gamma"])
def test_retention_full_size_slices_against_the_oracle(generated):
    """B=8 H=16 S=2048 Dqk=256 Dv=512 (the benchmark shape): three (batch, head) slices of the parallel operator against
    oracle.retention_parallel (bench_utils.py:1158-1163 restated) at atol 2e-2 / rtol 1e-2, the row scale r at 1e-3 --
    with the [1,H,S,S] multiplier tensor the reference's operator takes, and with the kernel generating it from gamma."""
    hb = _hb()
    B, H, S, D, DV = 8, 16, 2048, 256, 512
    q, k, v, _ = inputs.retnet_inputs(B, H, S, D, DV, seed=3, layout="bshd")
    q = (q.float() * 4.0).bfloat16()          # row sums straddle the clamp at 1
    mask32 = oracle.retention_decay_mask(H, S)                  # fp32 gamma_h^(i - j) [i >= j]
    rs = torch.full((B, H, S), float("nan"), device="cuda")
    print(f"retention full size, generated={generated}", flush=True)
    if generated:
        gamma = (1.0 - torch.exp2(-5.0 - torch.arange(H, dtype=torch.float64))).float()
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0, decay_gamma=gamma.cuda(),
                        row_scale=rs)
        ref_mask = mask32                                        # the kernel's factors are fp32
    else:
        o = hb.attn_fwd(q.cuda(), k.cuda(), v.cuda(), family=hb.MA_ATTN_RETENTION, causal=True, scale=1.0,
                        score_mask=mask32.bfloat16().cuda(), row_scale=rs)
        ref_mask = mask32.bfloat16()                             # the operator reads the rounded tensor
    torch.cuda.synchronize()
    assert torch.isfinite(o.float()).all() and torch.isfinite(rs).all()
    assert float(rs.min()) == 1.0 and float(rs.max()) > 1.0     # both sides of the clamp occur
    for b, h in [(0, 0), (7, 15), (3, 9)]:
        ref, r_ref = oracle.retention_parallel(q[b:b + 1, :, h:h + 1], k[b:b + 1, :, h:h + 1], v[b:b + 1, :, h:h + 1],
                                               ref_mask[:, h:h + 1], return_r=True)
        oracle.assert_close(o[b:b + 1, :, h:h + 1].float().cpu(), ref, rtol=RTOL, atol=ATOL)
        torch.testing.assert_close(rs[b:b + 1, h:h + 1].cpu(), r_ref, rtol=1e-3, atol=1e-3)
