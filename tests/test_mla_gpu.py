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


@pytest.mark.parametrize("B,Hq,page,pages_per_seq,dtype", [(4, 128, 64, 8, torch.bfloat16), (3, 16, 64, 5, torch.float16), (2, 40, 32, 9, torch.bfloat16)])
def test_paged_mla_with_kvcache(B, Hq, page, pages_per_seq, dtype):
    """flash_mla_with_kvcache-style call: fused 576-wide rows, shuffled page pool, ragged cache lengths."""
    hb = _hb()
    g = torch.Generator().manual_seed(B * 100 + Hq)
    npg = B * pages_per_seq + 3
    q = torch.randn(B, 1, Hq, 576, generator=g).to(dtype)
    cache = torch.randn(npg, page, 1, 576, generator=g).to(dtype)
    table = torch.randperm(npg, generator=g)[:B * pages_per_seq].to(torch.int32).view(B, pages_per_seq)
    lens = torch.randint(1, page * pages_per_seq + 1, (B,), generator=g, dtype=torch.int32)
    lens[0] = page * pages_per_seq
    meta, splits = hb.get_mla_metadata(lens.cuda(), Hq, 1)
    print(f"paged mla B{B} Hq{Hq} page{page} x{pages_per_seq} lens {lens.tolist()} {dtype}", flush=True)
    out, lse = hb.flash_mla_with_kvcache(q.cuda(), cache.cuda(), table.cuda(), lens.cuda(), 512, meta, splits)
    torch.cuda.synchronize()
    assert out.shape == (B, 1, Hq, 512) and lse.shape == (B, Hq, 1)
    ref, lse_ref = oracle.paged_mla_decode(q, cache, table, lens)
    oracle.assert_close(out.float().cpu(), ref, rtol=1e-2, atol=2e-2)
    torch.testing.assert_close(lse.cpu(), lse_ref, rtol=1e-4, atol=1e-4)


def test_mla_cache_lengths_without_pages():
    hb = _hb()
    B, Hq, Skv = 3, 128, 1024
    q, q_pe, kv, k_pe = inputs.mla_inputs(B, Hq, Skv, 512, 64, seed=4)
    lens = torch.tensor([1024, 700, 33], dtype=torch.int32)
    o = hb.mla_decode(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda(), scale=SCALE, kv_seqlens=lens.cuda())
    torch.cuda.synchronize()
    for b in range(B):
        L = int(lens[b])
        ref = oracle.mla_decode(q[b:b + 1], q_pe[b:b + 1], kv[b:b + 1, :L], k_pe[b:b + 1, :L])
        oracle.assert_close(o[b:b + 1].float().cpu(), ref, rtol=1e-2, atol=2e-2)


def test_engine_paged_mla_backend():
    """examples/mla_decode_v2.py through the engine: mod(q [B,1,Hq,576], KV [B*Skv/64, 64, 1, 576]) -> (out, lse)
    (testing/benchmark_h100.py:1079-1087)."""
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    import specs
    B, Hq, Skv = 2, 128, 512
    meta = (meta_tensor(B, Hq, 1, 576, dtype=torch.bfloat16), meta_tensor(B, 1, Skv, 576, dtype=torch.bfloat16),
            meta_tensor(B, 1, Skv, 512, dtype=torch.bfloat16))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=lambda s, io, b, h, q, k: s * (576 ** -0.5), mask_mod=None,
                          online_func=specs.OnlineSoftmax(), kv_shared=True, backend="cute")
    g = torch.Generator().manual_seed(6)
    q = torch.randn(B, 1, Hq, 576, generator=g).bfloat16()
    cache = torch.randn(B * Skv // 64, 64, 1, 576, generator=g).bfloat16()
    out, lse = mod(q.cuda(), cache.cuda())
    torch.cuda.synchronize()
    rows = cache.view(B, Skv, 1, 576)
    ref, lse_ref = oracle.mla_decode(q[..., :512], q[..., 512:], rows[..., :512], rows[..., 512:], return_lse=True)
    oracle.assert_close(out.float().cpu(), ref, rtol=1e-2, atol=2e-2)
    torch.testing.assert_close(lse.cpu()[:, :, 0], lse_ref, rtol=1e-4, atol=1e-4)


def test_engine_paged_mla_backend_ragged_length():
    """A cache length that is not a multiple of 256: the reference's block table gives sequence b the pages from
    b * pad / 64 on, pad = the length rounded up to 256 (attn_engine.py:211-216), so the pool is laid out that way;
    a pool too small for that layout is refused."""
    from attn_engine import AttentionEngine
    from core import CustomIO, meta_tensor
    import specs
    B, Hq, Skv, pad = 3, 128, 200, 256
    meta = (meta_tensor(B, Hq, 1, 576, dtype=torch.bfloat16), meta_tensor(B, 1, Skv, 576, dtype=torch.bfloat16),
            meta_tensor(B, 1, Skv, 512, dtype=torch.bfloat16))
    mod = AttentionEngine(meta, CustomIO({}), score_mod=lambda s, io, b, h, q, k: s * (576 ** -0.5), mask_mod=None,
                          online_func=specs.OnlineSoftmax(), kv_shared=True, backend="cute")
    g = torch.Generator().manual_seed(8)
    q = torch.randn(B, 1, Hq, 576, generator=g).bfloat16()
    cache = torch.randn(B * pad // 64, 64, 1, 576, generator=g).bfloat16()
    out, lse = mod(q.cuda(), cache.cuda())
    torch.cuda.synchronize()
    rows = cache.view(B, pad, 1, 576)[:, :Skv]
    ref, lse_ref = oracle.mla_decode(q[..., :512], q[..., 512:], rows[..., :512], rows[..., 512:], return_lse=True)
    oracle.assert_close(out.float().cpu(), ref, rtol=1e-2, atol=2e-2)
    torch.testing.assert_close(lse.cpu()[:, :, 0], lse_ref, rtol=1e-4, atol=1e-4)
    with pytest.raises(ValueError):
        mod(q.cuda(), cache[:B * Skv // 64].cuda())


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_mla_plan_kernel_matches_the_oracle(seed):
    """get_mla_metadata (cute_template_kvshared/kernels/get_mla_metadata.cu:8-75) is integer work: bit-exact."""
    hb = _hb()
    import numpy as np
    rng = np.random.default_rng(seed)
    for _ in range(12):
        B = int(rng.integers(1, 70))
        lens = rng.integers(0, 9000, size=B).astype(np.int32)
        if rng.random() < 0.3:
            lens[:] = int(rng.integers(1, 5000))
        parts = int(rng.choice([1, 2, 7, 64, 128, 256, 300]))
        meta, splits = hb.get_mla_metadata(torch.from_numpy(lens).cuda(), 128, 1, num_sm_parts=parts)
        torch.cuda.synchronize()
        ref_meta, ref_splits = oracle.mla_work_plan(lens, parts)
        assert meta.shape == (parts, 8) and np.array_equal(meta.cpu().numpy(), ref_meta), (B, parts, lens.tolist())
        assert np.array_equal(splits.cpu().numpy(), ref_splits)
    assert hb.get_mla_metadata(torch.ones(3, dtype=torch.int32, device="cuda"), 128, 1)[0].shape[0] == hb.load_library().ma_mla_num_sm_parts(128)


@pytest.mark.parametrize("B,Hq,parts,maxlen", [(24, 128, 0, 4096), (5, 128, 7, 3000), (3, 64, 256, 700), (1, 128, 256, 32768)])
def test_planned_paged_mla_decode(B, Hq, parts, maxlen):
    """Ragged batches through the work plan: every workgroup walks the pieces of its part (batch entries cut at part
    boundaries are merged by the combine kernel; the last case cuts one long sequence into more than 64 pieces).  Same
    results as the paged oracle, and as the launch without a plan up to the rounding of the partial outputs."""
    hb = _hb()
    page = 64
    g = torch.Generator().manual_seed(B + maxlen)
    pages_per_seq = (maxlen + page - 1) // page
    npg = B * pages_per_seq + 2
    q = torch.randn(B, 1, Hq, 576, generator=g).bfloat16()
    cache = torch.randn(npg, page, 1, 576, generator=g).bfloat16()
    table = torch.randperm(npg, generator=g)[:B * pages_per_seq].to(torch.int32).view(B, pages_per_seq)
    lens = torch.randint(1, maxlen + 1, (B,), generator=g, dtype=torch.int32)
    lens[0] = maxlen
    if B > 2:
        lens[1] = 0            # an empty cache entry: zeros, lse = -inf
        lens[2] = 1
    meta, splits = hb.get_mla_metadata(lens.cuda(), Hq, 1, num_sm_parts=parts)
    print(f"planned mla B{B} Hq{Hq} parts{meta.shape[0]} pieces {int(splits[-1])} lens {lens.tolist()[:8]}..", flush=True)
    out, lse = hb.flash_mla_with_kvcache(q.cuda(), cache.cuda(), table.cuda(), lens.cuda(), 512, meta, splits)
    out_u, lse_u = hb.flash_mla_with_kvcache(q.cuda(), cache.cuda(), table.cuda(), lens.cuda(), 512)
    torch.cuda.synchronize()
    if B == 1:
        assert int(splits[-1]) > 64
    check = list(range(B)) if B <= 6 else [0, 1, 2, 3, B - 1]
    for b in check:
        if int(lens[b]) == 0:
            assert torch.count_nonzero(out[b]) == 0 and torch.isinf(lse[b]).all() and (lse[b] < 0).all()
            continue
        ref, lse_ref = oracle.paged_mla_decode(q[b:b + 1], cache, table[b:b + 1], lens[b:b + 1])
        oracle.assert_close(out[b:b + 1].float().cpu(), ref, rtol=1e-2, atol=2e-2)
        torch.testing.assert_close(lse[b:b + 1].cpu(), lse_ref, rtol=1e-4, atol=1e-4)
    # the launch without a plan: same results, empty entries included (zeros and lse = -inf from its combine kernel too)
    torch.testing.assert_close(out.float(), out_u.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(lse, lse_u, rtol=1e-4, atol=1e-4)
    assert torch.isfinite(out_u.float()).all()


@pytest.mark.parametrize("num_split", [0, 1, 3, 8])
def test_mla_decode_with_an_empty_cache_entry(num_split):
    """kv_seqlens with a zero in it through the uniform launch, unsplit and split: that batch entry gets zeros and
    lse = -inf (every piece of it is empty, so the combine kernel has nothing to weigh), the others are unaffected."""
    hb = _hb()
    B, Hq, Skv = 4, 128, 640
    q, q_pe, kv, k_pe = inputs.mla_inputs(B, Hq, Skv, 512, 64, seed=3)
    lens = torch.tensor([Skv, 0, 37, 300], dtype=torch.int32)
    lse = torch.full((B, Hq), float("nan"), device="cuda")
    o = hb.mla_decode(q.cuda(), q_pe.cuda(), kv.cuda(), k_pe.cuda(), scale=SCALE, num_split=num_split, lse=lse,
                      kv_seqlens=lens.cuda())
    torch.cuda.synchronize()
    assert torch.count_nonzero(o[1]) == 0 and torch.isinf(lse[1]).all() and (lse[1] < 0).all()
    for b in (0, 2, 3):
        n = int(lens[b])
        ref, lse_ref = oracle.mla_decode(q[b:b + 1], q_pe[b:b + 1], kv[b:b + 1, :n], k_pe[b:b + 1, :n], return_lse=True)
        oracle.assert_close(o[b:b + 1].float().cpu(), ref, rtol=1e-2, atol=2e-2)
        torch.testing.assert_close(lse[b:b + 1].cpu(), lse_ref.view(1, Hq), rtol=1e-4, atol=1e-4)
