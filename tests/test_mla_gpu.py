"""Parity of the HIP MLA decode (split-KV + combine, through the C ABI) with
the CPU oracle.  Tolerance atol 2e-2 / rtol 1e-2 (fp32-accumulated bf16)."""
import math

import pytest
import torch

import oracle
from oracle import inputs

pytestmark = pytest.mark.gpu
SCALE = 1 / math.sqrt(576)


def _hb():
    from metaattention_amd import hip_backend as hb
    hb.load_library()
    return hb


@pytest.mark.parametrize("B,Hq,Skv,ns", [
    (1, 64, 64, 1), (2, 128, 256, 1), (2, 128, 256, 2), (1, 16, 100, 1), (3, 40, 1000, 3),
    (8, 128, 2048, 0), (1, 128, 333, 4), (1, 1, 1, 1), (2, 7, 65, 2), (1, 128, 4096, 0),
])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_mla_decode(B, Hq, Skv, ns, dtype):
    hb = _hb()
    q, q_pe, kv, k_pe = inputs.mla_inputs(B, Hq, Skv, 512, 64, dtype=dtype, seed=Skv)
    ref, lse_ref = oracle.mla_decode(q, q_pe, kv, k_pe, return_lse=True)
    lse = torch.full((B, Hq), float("nan"), device="cuda")
    print(f"mla B{B} Hq{Hq} Skv{Skv} ns{ns} {dtype}", flush=True)
    o = hb.mla_decode(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda(), scale=SCALE, num_split=ns, lse=lse)
    torch.cuda.synchronize()
    oracle.assert_close(o.float().cpu(), ref, rtol=1e-2, atol=2e-2)
    torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-4, atol=1e-4)


def test_mla_split_invariance_full_size():
    """Benchmark shape (B=64, Hq=128, Skv=4096): the result must not depend on the
    number of kv splits beyond fp32 merge rounding, and a few batch entries must match the oracle."""
    hb = _hb()
    B, Hq, Skv = 64, 128, 4096
    g = torch.Generator(device="cuda").manual_seed(0)
    q = torch.randn(B, 1, Hq, 512, device="cuda", dtype=torch.bfloat16, generator=g)
    q_pe = torch.randn(B, 1, Hq, 64, device="cuda", dtype=torch.bfloat16, generator=g)
    kv = torch.randn(B, Skv, 1, 512, device="cuda", dtype=torch.bfloat16, generator=g)
    k_pe = torch.randn(B, Skv, 1, 64, device="cuda", dtype=torch.bfloat16, generator=g)
    outs = [hb.mla_decode(q, q_pe, kv, k_pe, scale=SCALE, num_split=ns) for ns in (1, 2, 8)]
    torch.cuda.synchronize()
    for o in outs[1:]:
        torch.testing.assert_close(o.float(), outs[0].float(), rtol=1e-2, atol=2e-3)
    for b in (0, 37, 63):
        ref = oracle.mla_decode(q[b:b + 1].cpu(), q_pe[b:b + 1].cpu(), kv[b:b + 1].cpu(), k_pe[b:b + 1].cpu())
        oracle.assert_close(outs[1][b:b + 1].float().cpu(), ref, rtol=1e-2, atol=2e-2)


def test_mla_through_engine():
    import specs
    B, Hq, Skv = 2, 128, 512
    mod = specs.mla_decode(B, Hq, Skv, 576, 512)
    q, q_pe, kv, k_pe = inputs.mla_inputs(B, Hq, Skv, 512, 64, seed=11)
    o = mod(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda())
    torch.cuda.synchronize()
    assert o.shape == (B, 1, Hq, 512)
    oracle.assert_close(o.float().cpu(), oracle.mla_decode(q, q_pe, kv, k_pe), rtol=1e-2, atol=2e-2)


def test_mla_rejects_bad_arguments():
    hb = _hb()
    q = torch.zeros(1, 1, 16, 256, device="cuda", dtype=torch.bfloat16)
    qp = torch.zeros(1, 1, 16, 64, device="cuda", dtype=torch.bfloat16)
    kv = torch.zeros(1, 64, 1, 256, device="cuda", dtype=torch.bfloat16)
    kp = torch.zeros(1, 64, 1, 64, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(hb.MetaAttentionError) as ei:
        hb.mla_decode(q, qp, kv, kp, scale=SCALE)
    assert "dim=512" in str(ei.value)
    q5 = torch.zeros(1, 1, 16, 512, device="cuda", dtype=torch.bfloat16)
    kv5 = torch.zeros(1, 64, 1, 512, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(hb.MetaAttentionError):
        hb.mla_decode(q5, qp, kv5, kp, scale=SCALE, num_split=5)     # more splits than kv tiles
