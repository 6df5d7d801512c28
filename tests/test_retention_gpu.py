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
